/*
 * qmlp_hip.h -- the thin C ABI through which the QuickMLP host code reaches the GPU.
 *
 * It replaces the runtime compile/launch loader the reference links against
 * (third-party/cuda-kernel-loader, an NVRTC + CUDA-driver wrapper whose source is not
 * vendored; its API is visible at the reference's call sites, cited per function below)
 * and the few CUDA runtime calls the reference's host code makes directly.
 *
 * Conventions: every function returns 0 on success and a non-zero code on failure;
 * qmlp_hip_last_error() then returns a thread-local, human-readable message. Handles
 * are opaque. No C++ or torch type crosses this boundary. All kernels are gfx950 code
 * objects compiled at run time with hipRTC; compiling needs no GPU, loading does.
 */
#ifndef QMLP_HIP_H
#define QMLP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qmlp_hip_module_s* qmlp_hip_module;
typedef struct qmlp_hip_function_s* qmlp_hip_function;
typedef void* qmlp_hip_stream;   /* a hipStream_t; NULL = the default stream */
typedef void* qmlp_hip_event;    /* a hipEvent_t */

typedef struct {
    int wave_size;               /* 64 on CDNA */
    int compute_units;
    int lds_bytes_per_block;     /* 163840 on gfx950 */
    int max_threads_per_block;
    int clock_khz;
    size_t total_memory;
    char arch[64];               /* e.g. "gfx950:sramecc+:xnack-" */
} qmlp_hip_device_props;

/* Message of the last failing call on this thread ("" if none). */
const char* qmlp_hip_last_error(void);

/* Replaces ckl::KernelLoader::isCudaAvailable / checkCudaAvailable
 * (src_cpp/src/qmlp.cpp:41-49). count = 0 when no usable GPU is present. */
int qmlp_hip_device_count(int* count);
/* Replaces cudaGetDeviceProperties (src_cpp/src/fused_network.cpp:12-31). */
int qmlp_hip_get_device_props(int device, qmlp_hip_device_props* props);

/* Replace cudaMalloc/cudaFree/cudaMemset/cudaMemcpy[Async]
 * (src_cpp/src/tensor.cpp:41-44,68-98, include/qmlp/tmp_memory.h:14-36). */
int qmlp_hip_malloc(void** ptr, size_t bytes);
int qmlp_hip_free(void* ptr);
int qmlp_hip_memset_async(void* ptr, int value, size_t bytes, qmlp_hip_stream stream);
int qmlp_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, qmlp_hip_stream stream);
int qmlp_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, qmlp_hip_stream stream);
int qmlp_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, qmlp_hip_stream stream);
int qmlp_hip_device_synchronize(void);

/* Replace cudaStreamCreateWithFlags / cudaEventCreateWithFlags / cudaEventRecord /
 * cudaStreamWaitEvent (src_cpp/src/fused_network.cpp:208-235,1076-1078,1110-1142).
 * Streams are created non-blocking at the default priority. */
int qmlp_hip_stream_create(qmlp_hip_stream* stream);
int qmlp_hip_stream_destroy(qmlp_hip_stream stream);
int qmlp_hip_stream_synchronize(qmlp_hip_stream stream);
int qmlp_hip_event_create(qmlp_hip_event* event, int enable_timing);
int qmlp_hip_event_destroy(qmlp_hip_event event);
int qmlp_hip_event_record(qmlp_hip_event event, qmlp_hip_stream stream);
int qmlp_hip_event_synchronize(qmlp_hip_event event);
int qmlp_hip_stream_wait_event(qmlp_hip_stream stream, qmlp_hip_event event);
int qmlp_hip_event_elapsed_ms(qmlp_hip_event start, qmlp_hip_event stop, float* ms);

/* Replaces ckl::KernelLoader::getKernel(name, source, constants, flags)
 * (src_cpp/src/fused_network.cpp:465-470,949-953): compiles `source` with hipRTC for
 * `arch` (NULL: the current device, or gfx950 when there is none). `headers` /
 * `header_names` are in-memory include files. `name_expressions` are C++ names of
 * __global__ functions (template instantiations allowed) whose lowered names can be
 * queried afterwards. On failure the compiler log is part of the error message.
 * If `log` is non-NULL it receives a malloc'ed copy of the log (free with
 * qmlp_hip_free_string). */
int qmlp_hip_module_compile(const char* source, const char* source_name,
                            const char* const* header_names, const char* const* headers,
                            int num_headers,
                            const char* const* name_expressions, int num_expressions,
                            const char* const* options, int num_options,
                            const char* arch,
                            qmlp_hip_module* module, char** log);
void qmlp_hip_free_string(char* s);
/* What qmlp_hip_module_compile(..., arch, ...) compiles for and with: "<architecture>;hiprtc <major>.<minor>",
 * the architecture resolved as there (arch, else the current device, else gfx950) and cut at the first ':'. Part of the key of the
 * on-disk kernel cache (the reference's ckl::KernelLoader keys its cache on source and flags only,
 * third-party/cuda-kernel-loader as used in src_cpp/src/qmlp.cpp:23-35). Returns a malloc'ed string
 * (free with qmlp_hip_free_string) through `target`. */
int qmlp_hip_compile_target(const char* arch, char** target);
/* Wraps an existing code object (e.g. from the on-disk kernel cache). */
int qmlp_hip_module_from_code(const void* code, size_t size, qmlp_hip_module* module);
int qmlp_hip_module_code(qmlp_hip_module module, const void** code, size_t* size);
/* Lowered (mangled) name of a name expression given to qmlp_hip_module_compile. */
int qmlp_hip_module_lowered_name(qmlp_hip_module module, const char* name_expression,
                                 const char** lowered);
/* Loads the code object onto the current device (needs a GPU; idempotent). */
int qmlp_hip_module_load(qmlp_hip_module module);
int qmlp_hip_module_destroy(qmlp_hip_module module);
/* Replaces the KernelFunction handle (fun.call / fun.name / fun.defined). The function
 * handle is owned by its module. */
int qmlp_hip_module_get_function(qmlp_hip_module module, const char* lowered_name,
                                 qmlp_hip_function* function);
/* Replaces ckl::KernelFunction::constant(name) (src_cpp/src/encoding_hashgrid.cpp:241). */
int qmlp_hip_module_get_global(qmlp_hip_module module, const char* name, void** device_ptr,
                               size_t* bytes);
/* Replaces KernelFunction::bestBlockSize()/minGridSize()
 * (src_cpp/src/fused_network.cpp:473,540). */
int qmlp_hip_function_occupancy(qmlp_hip_function function, size_t dynamic_lds_bytes,
                                int block_size_limit, int* block_size, int* min_grid_size);
/* Workgroups of block_size threads (with dynamic_lds_bytes of dynamic LDS each) that one
 * compute unit holds at the same time; what the grid of a persistent kernel is sized with.
 * No counterpart in cuda-kernel-loader (the reference sizes grids with minGridSize()). */
int qmlp_hip_function_blocks_per_cu(qmlp_hip_function function, int block_size, size_t dynamic_lds_bytes,
                                    int* blocks_per_cu);
/* Register / LDS usage of a loaded function (for logging and launch sizing). */
int qmlp_hip_function_attributes(qmlp_hip_function function, int* num_vgprs, int* static_lds_bytes,
                                 int* max_threads_per_block, int* scratch_bytes);
/* Replaces KernelFunction::call(grid, block, shared, stream, args...)
 * (src_cpp/src/fused_network.cpp:548-550). `args` holds one pointer per kernel
 * parameter, as for hipModuleLaunchKernel. */
int qmlp_hip_launch(qmlp_hip_function function, unsigned grid_x, unsigned block_x,
                    unsigned dynamic_lds_bytes, qmlp_hip_stream stream, void** args);

#ifdef __cplusplus
}
#endif
#endif
