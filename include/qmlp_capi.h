/*
 * qmlp_capi.h -- C ABI of the fused encoding + MLP operators.
 *
 * These entry points are what a foreign-function binding of QuickMLP binds; each one
 * maps 1:1 onto a method of the reference's C++ API (class qmlp::FusedNetwork,
 * qmlp::IEncoding, qmlp::Activation, qmlp::QuickMLP), the same set its PyTorch binding
 * exposes through TORCH_LIBRARY (src_cpp/pytorch-bindings/src/bind_network.cpp:346-411,
 * bind_encoding.cpp:165-197, bind_activation.cpp:80-98, bindings.cpp:102-122). Reference
 * locations are given per function as file:line below the reference's root.
 *
 * Conventions: plain pointers and sizes only. Every function returns 0 on success and
 * non-zero on failure; qmlp_last_error() then holds the message (C++ exceptions never
 * cross the boundary: 1 = configuration error, 2 = runtime/shape/type error,
 * 3 = device/compiler error). Tensors are described by qmlp_tensor: a device pointer the
 * caller owns plus shape and strides in elements. All work is enqueued on the given
 * HIP stream (NULL = default stream). Gradients are accumulated (+=): the caller zeroes.
 * Objects are stateful (current parameter tensors) and not thread-safe.
 */
#ifndef QMLP_CAPI_H
#define QMLP_CAPI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct qmlp_network_s* qmlp_network_t;
typedef struct qmlp_encoding_s* qmlp_encoding_t;
typedef struct qmlp_activation_s* qmlp_activation_t;

/* qmlp::Tensor::Precision / ::Usage (src_cpp/include/qmlp/tensor.h:25-38) */
enum { QMLP_FLOAT = 0, QMLP_HALF = 1, QMLP_DOUBLE = 2 };
enum { QMLP_INFERENCE = 0, QMLP_GRADIENTS = 1 };
/* qmlp::FusedNetwork::AdjointMode (src_cpp/include/qmlp/fused_network.h:22-33) */
enum { QMLP_GRADIENTS_INPUT = 1, QMLP_GRADIENTS_NETWORK_WEIGHTS = 2, QMLP_GRADIENTS_INPUT_ENCODINGS = 4 };
/* qmlp::IEncoding::AdjointMode (src_cpp/include/qmlp/iencoding.h:112-117) */
enum { QMLP_ENCODING_INPUT_GRADIENTS = 1, QMLP_ENCODING_PARAM_GRADIENTS = 2 };

/* Non-owning strided tensor: the C form of qmlp::Tensor(void*, precision, sizes, strides)
 * (src_cpp/include/qmlp/tensor.h:79-85). ndim = 0 means "undefined". */
typedef struct {
    void* data;
    int32_t precision;
    int32_t ndim;
    int32_t sizes[4];
    int32_t strides[4];
} qmlp_tensor;

const char* qmlp_last_error(void);
/* Frees strings returned through char** parameters. */
void qmlp_free_string(char* s);

/* ---- qmlp::QuickMLP singleton (src_cpp/include/qmlp/qmlp.h:14-94) ---- */
int qmlp_is_gpu_available(int* available);                 /* isCudaAvailable, qmlp.h:38 */
int qmlp_set_log_level(const char* level_name);             /* setLogLevel(name), qmlp.h:71 */
int qmlp_set_compile_debug_mode(int enable);                /* setCompileDebugMode, qmlp.h:85 */
int qmlp_is_compile_debug_mode(int* enabled);               /* isCompileDebugMode, qmlp.h:87 */
/* Kernel cache control: ckl setCacheDir / disableCudaCache (src_cpp/src/qmlp.cpp:17,
 * tests_cpp/main.cpp:30-31). NULL or "" disables the disk cache. */
int qmlp_set_kernel_cache_dir(const char* directory);
/* Number of runtime compilations / disk-cache hits so far (diagnostics). */
int qmlp_kernel_cache_stats(int* compilations, int* disk_hits);
/* Whether kernels without template arguments that ask for it are compiled by the offline compiler of the installed
 * ROCm (<ROCM_PATH>/bin/hipcc as a child process; QMLP_COMPILER=hiprtc in the environment switches it off) instead of
 * the run-time compiler that the process has loaded, and how many were so far. No counterpart in the reference
 * (its loader only has NVRTC); diagnostics for tests and logs. */
int qmlp_kernel_compiler_stats(int* has_offline_compiler, int* offline_compilations);

/* ---- qmlp::FusedNetwork (src_cpp/include/qmlp/fused_network.h:16-338) ---- */
/* FusedNetwork(cfg, parent), fused_network.h:157 / src_cpp/src/fused_network.cpp:33-223 */
int qmlp_network_create(const char* cfg_json, const char* parent_directory, qmlp_network_t* network);
int qmlp_network_destroy(qmlp_network_t network);
int qmlp_network_channels_in(qmlp_network_t network, int* value);          /* channelsIn, :164 */
int qmlp_network_channels_out(qmlp_network_t network, int* value);         /* channelsOut, :165 */
int qmlp_network_num_layers(qmlp_network_t network, int* value);           /* numLayers, :168 */
int qmlp_network_num_encodings(qmlp_network_t network, int* value);        /* numEncodings, :161 */
/* encoding(idx), :162. The handle is borrowed: valid while the network lives, do not destroy. */
int qmlp_network_encoding(qmlp_network_t network, int index, qmlp_encoding_t* encoding);
int qmlp_network_parameter_count(qmlp_network_t network, int* value);      /* networkParameterCount, :170 */
int qmlp_network_parameter_precision(qmlp_network_t network, int usage, int* precision); /* :172 */
int qmlp_network_matrix_size(int* value);                                  /* MATRIX_SIZE, :142 */
int qmlp_network_warp_size(int* value);                                    /* WARP_SIZE, :145 */
int qmlp_network_max_shared_memory_bytes(int* value);                      /* MAX_SHARED_MEMORY_BYTES, :148 */
int qmlp_network_is_parallel_streams(qmlp_network_t network, int* value);  /* bind_network.h:52 */
int qmlp_network_set_parallel_streams(qmlp_network_t network, int enabled);
/* setNetworkParameter(tensor, usage), :180. An undefined tensor clears the binding. */
int qmlp_network_set_parameter(qmlp_network_t network, const qmlp_tensor* tensor, int usage);
/* initializeInferenceParameters(rng), :188, with std::default_random_engine(seed). */
int qmlp_network_initialize_inference_parameters(qmlp_network_t network, uint32_t seed);
/* networkParameter(layer, bias, rawPtr, precision), :205: view into a flat parameter
 * tensor; `view->ndim` = 0 if the layer has no bias. */
int qmlp_network_parameter_view(qmlp_network_t network, int layer, int bias, void* raw_pointer,
                                int precision, qmlp_tensor* view);
/* inference(input, output, stream), :229 */
int qmlp_network_inference(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* output,
                           void* stream);
/* qmlp_network_inference for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc); it has no counterpart in the
 * reference. Same arguments and the same results bit for bit, but no call on its way
 * allocates or frees: the workspace in which a batch is ordered by grid slab (networks with a
 * large dense grid; qmlp_network_inference keeps one per network and allocates it on demand)
 * is a static device buffer of 48 MiB per GPU, and kernels are only used if they are
 * loaded already. So: run qmlp_network_inference once on a batch of the same size first
 * (that compiles and loads the kernels and resolves the buffer on this GPU). Errors:
 * a batch whose order needs more than the buffer (20.5 bytes per point at 4 input channels:
 * about 2.4 million points), kernels that are not loaded yet. All calls on one GPU share the
 * buffer, whose contents are not kept between calls: calls that overlap in time race. */
int qmlp_network_inference_noalloc(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* output,
                                   void* stream);
/* forwardMemory(numElements, flags), :240 */
int qmlp_network_forward_memory(qmlp_network_t network, int num_elements, int adjoint_flags, size_t* bytes);
/* forward(input, output, tmpMemory, stream), :263 */
int qmlp_network_forward(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* output,
                         void* tmp_memory, void* stream);
/* zeroGradients(), :269 */
int qmlp_network_zero_gradients(qmlp_network_t network);
/* adjointMemory(numElements, flags), :280 */
int qmlp_network_adjoint_memory(qmlp_network_t network, int num_elements, int adjoint_flags, size_t* bytes);
/* adjoint(input, adjOutput, flags, adjInput, tmpFwd, tmpAdj, stream), :313.
 * adj_input may be NULL / undefined unless QMLP_GRADIENTS_INPUT is set. */
int qmlp_network_adjoint(qmlp_network_t network, const qmlp_tensor* input, const qmlp_tensor* adj_output,
                         int adjoint_flags, const qmlp_tensor* adj_input, const void* tmp_memory_forward,
                         void* tmp_memory_adjoint, void* stream);
/* clearCachedKernels(), :319 */
int qmlp_network_clear_cached_kernels(qmlp_network_t network);
/* Generates and compiles all kernels of the network without touching a GPU
 * (adjoint_flags <= 0: inference and forward only). No counterpart in the reference,
 * where kernels can only be compiled with a device present. */
int qmlp_network_precompile(qmlp_network_t network, int adjoint_flags);
/* Loads the kernels that calls on a batch of `numel` points take (inference; forward and adjoint too if
 * adjoint_flags > 0) and allocates the workspace that orders such a batch by grid slab, so that the calls
 * themselves only enqueue kernels (for callers that capture them into a HIP graph). No counterpart in the
 * reference, whose first call on a network compiles its kernels. */
int qmlp_network_prepare(qmlp_network_t network, int numel, int adjoint_flags);
/* The generated device source; kind = "inference" | "forward" | "backward" | "weight_update". Diagnostics as JSON:
 * "shapes" (the shapes of the forward kernel the network may launch), "backward_resources" and
 * "backward_slices_resources" (workgroup size, LDS, registers and scratch bytes of the loaded backward kernel;
 * these two need a device). */
int qmlp_network_generated_source(qmlp_network_t network, const char* kind, int adjoint_flags, char** source);

/* ---- qmlp::IEncoding (src_cpp/include/qmlp/iencoding.h:36-140) ---- */
/* EncodingFactory::Instance().create(cfg), iencoding.h:190-200 */
int qmlp_encoding_create(const char* cfg_json, qmlp_encoding_t* encoding);
int qmlp_encoding_destroy(qmlp_encoding_t encoding);
int qmlp_encoding_to_json(qmlp_encoding_t encoding, char** json);                 /* toJson, :41 */
int qmlp_encoding_id(qmlp_encoding_t encoding, char** id);                        /* id, :42 */
int qmlp_encoding_max_input_channel(qmlp_encoding_t encoding, int* value);        /* :48 */
int qmlp_encoding_num_output_channels(qmlp_encoding_t encoding, int* value);      /* :53 */
int qmlp_encoding_has_parameters(qmlp_encoding_t encoding, int* value);           /* :73 */
int qmlp_encoding_parameter_count(qmlp_encoding_t encoding, int* value);          /* :82 */
int qmlp_encoding_parameter_precision(qmlp_encoding_t encoding, int usage, int* precision); /* :80 */
int qmlp_encoding_set_parameter(qmlp_encoding_t encoding, const qmlp_tensor* tensor, int usage); /* :90 */
int qmlp_encoding_zero_gradients(qmlp_encoding_t encoding);                       /* :104 */
/* forward(input, output, stream, parametersForward), :115 (parameters may be NULL) */
int qmlp_encoding_forward(qmlp_encoding_t encoding, const qmlp_tensor* input, const qmlp_tensor* output,
                          void* stream, const qmlp_tensor* parameters_forward);
/* adjoint(input, adjOutput, adjInput, stream, paramsFwd, paramsGrad, mode), :132 */
int qmlp_encoding_adjoint(qmlp_encoding_t encoding, const qmlp_tensor* input, const qmlp_tensor* adj_output,
                          const qmlp_tensor* adj_input, void* stream, const qmlp_tensor* parameters_forward,
                          const qmlp_tensor* parameters_gradients, int adjoint_mode);
/* Compiles the standalone kernels (forward, and the adjoint of adjoint_mode if > 0) into the
 * kernel cache without a GPU. No counterpart in the reference, which compiles lazily inside
 * forward()/adjoint() (src_cpp/src/iencoding.cpp:30-43,98-112). */
int qmlp_encoding_precompile(qmlp_encoding_t encoding, int adjoint_mode);
/* HashGrid only: level table as the reference computes it in
 * src_cpp/src/encoding_hashgrid.cpp:63-96. Arrays hold `capacity` entries. */
int qmlp_encoding_hashgrid_levels(qmlp_encoding_t encoding, int capacity, int* num_levels, int* memory_offset,
                                  int* resolution, int* hash_grid_size, int* hashed);
/* HashGrid only (test aid): runs the device index code and writes, for every point,
 * level and corner, the table offset of feature 0 and the interpolation weight:
 * indices/weights are device arrays of N * levels * 2^dim entries. */
int qmlp_encoding_hashgrid_corners(qmlp_encoding_t encoding, const qmlp_tensor* input, uint32_t* indices,
                                   float* weights, void* stream);
/* HashGrid only (test aid, no counterpart in the reference): the same two arrays, written by the
 * code the fused kernels run. mode 1: the table entries (element offset of feature 0) and weights
 * that the gathers of the fused forward / inference kernels use, including their paired loads
 * (needs a bound table, src_cpp/include/qmlp/kernels/encoding_hashgrid.cuh:267-336 is what they
 * replace); mode 2: the entries and weights the gradient scatter of the fused backward kernel
 * adds to (encoding_hashgrid.cuh:345-369; nothing is added); mode 3: the entries and weights that
 * the gradient records of large batches stand for (slice of the record's bucket + 16-bit offsets,
 * and the entries of other slices that the records kernel adds itself; grids that offer gradient
 * slices only); mode 4: the entries behind the sums of the column kernel of sorted batches (the place of
 * each corner in the LDS of the owner of its node, and back to the table as the kernel writes its sums;
 * single dense levels that offer gradient columns only); mode 0 = qmlp_encoding_hashgrid_corners.
 * The order of the 2^dim corners of a level is the order the code visits them. input = NULL only
 * compiles the kernel of that mode into the kernel cache (needs no GPU). */
int qmlp_encoding_hashgrid_trace(qmlp_encoding_t encoding, const qmlp_tensor* input, int mode, uint32_t* indices,
                                 float* weights, void* stream);

/* ---- qmlp::Activation (src_cpp/include/qmlp/activation.h:29-150) ---- */
/* ActivationFactory(loader).getOrInline(key), activation.h:136: a built-in id or an inline
 * JSON object {"id","forward","adjoint"}. */
int qmlp_activation_create(const char* key_or_json, qmlp_activation_t* activation);
int qmlp_activation_destroy(qmlp_activation_t activation);
int qmlp_activation_to_json(qmlp_activation_t activation, char** json);           /* toJson, :41 */
int qmlp_activation_forward(qmlp_activation_t activation, const qmlp_tensor* input, const qmlp_tensor* output,
                            void* stream);                                         /* forward, :81 */
int qmlp_activation_adjoint(qmlp_activation_t activation, const qmlp_tensor* input, const qmlp_tensor* adj_output,
                            const qmlp_tensor* adj_input, void* stream);           /* adjoint, :92 */
/* Compiles the standalone kernels into the kernel cache without a device (the reference
 * compiles them on first use, src_cpp/src/activation.cpp:64-100). */
int qmlp_activation_precompile(qmlp_activation_t activation);

/* ---- qmlp::Utils (src_cpp/include/qmlp/utils.h:50-85; bound for torch as utils.pullpush_forward
 * and utils.pullpush_backward in src_cpp/pytorch-bindings/src/bind_utils.cpp:9-40) ---- */
/* fractionalPullpush, utils.h:65: mask (B,H,W), data and output (B,C,H,W), C < 16, all float
 * or all double. Returns after the work on 'stream' has finished (the image pyramid is
 * temporary device memory of the call). */
int qmlp_utils_pullpush_forward(const qmlp_tensor* mask, const qmlp_tensor* data, const qmlp_tensor* output,
                                void* stream);
/* adjointFractionalPullpush, utils.h:80: adds into adj_mask (B,H,W) and adj_data (B,C,H,W),
 * which the caller zeroes first (bind_utils.cpp:26-27). */
int qmlp_utils_pullpush_adjoint(const qmlp_tensor* mask, const qmlp_tensor* data, const qmlp_tensor* adj_output,
                                const qmlp_tensor* adj_mask, const qmlp_tensor* adj_data, void* stream);
/* Compiles the pull-push kernels for QMLP_FLOAT or QMLP_DOUBLE into the kernel cache without a
 * device (the reference compiles them on first use, src_cpp/src/utils.cpp:12-35 and :145-180). */
int qmlp_utils_pullpush_precompile(int precision);

#ifdef __cplusplus
}
#endif
#endif
