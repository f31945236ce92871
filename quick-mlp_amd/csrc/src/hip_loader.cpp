// Implementation of the thin C ABI in include/qmlp_hip.h on top of the HIP runtime,
// the HIP module API and hipRTC. Together with device_code.hip (the fill kernel and the
// static scratch buffer) these are the only translation units of the library that talk to HIP.
#include "qmlp_hip.h"
#include "qmlp/device_code.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local std::string g_lastError;

int fail(const std::string& msg)
{
    g_lastError = msg;
    return 1;
}

int check(hipError_t e, const char* what)
{
    if (e == hipSuccess) return 0;
    return fail(std::string(what) + ": " + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ")");
}

int checkRtc(hiprtcResult r, const char* what, const std::string& extra = "")
{
    if (r == HIPRTC_SUCCESS) return 0;
    std::string m = std::string(what) + ": " + hiprtcGetErrorString(r);
    if (!extra.empty()) m += "\n" + extra;
    return fail(m);
}

} // namespace

struct qmlp_hip_function_s
{
    hipFunction_t fn = nullptr;
    std::string name;
};

struct qmlp_hip_module_s
{
    std::vector<char> code;
    std::map<std::string, std::string> lowered;
    hipModule_t module = nullptr;
    bool loaded = false;
    std::map<std::string, qmlp_hip_function_s*> functions;
    std::mutex mutex;
};

extern "C" {

const char* qmlp_hip_last_error(void) { return g_lastError.c_str(); }

int qmlp_hip_device_count(int* count)
{
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e != hipSuccess) {
        (void)hipGetLastError();   // no device / no driver is not an error here
        c = 0;
    }
    *count = c;
    return 0;
}

int qmlp_hip_get_device_props(int device, qmlp_hip_device_props* props)
{
    hipDeviceProp_t p;
    if (int rc = check(hipGetDeviceProperties(&p, device), "hipGetDeviceProperties")) return rc;
    std::memset(props, 0, sizeof(*props));
    props->wave_size = p.warpSize;
    props->compute_units = p.multiProcessorCount;
    props->lds_bytes_per_block = static_cast<int>(p.sharedMemPerBlock);
    props->max_threads_per_block = p.maxThreadsPerBlock;
    props->clock_khz = p.clockRate;
    props->total_memory = p.totalGlobalMem;
    std::snprintf(props->arch, sizeof(props->arch), "%s", p.gcnArchName);
    return 0;
}

int qmlp_hip_malloc(void** ptr, size_t bytes)
{
    *ptr = nullptr;
    if (bytes == 0) return 0;
    return check(hipMalloc(ptr, bytes), "hipMalloc");
}

int qmlp_hip_free(void* ptr)
{
    if (!ptr) return 0;
    return check(hipFree(ptr), "hipFree");
}

int qmlp_hip_memset_async(void* ptr, int value, size_t bytes, qmlp_hip_stream stream)
{
    // a kernel, not hipMemsetAsync: memset nodes in a captured HIP graph have given wrong
    // results on replay on MI355X, and every call of the library is meant to be capturable
    std::string error;
    if (qmlp::device_code::fillAsync(ptr, value, bytes, stream, error) != 0) return fail(error);
    return 0;
}

int qmlp_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, qmlp_hip_stream stream)
{
    if (bytes == 0) return 0;
    if (int rc = check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice,
                                      static_cast<hipStream_t>(stream)), "hipMemcpyAsync(H2D)")) return rc;
    // the host buffer may be pageable and short-lived: finish before returning
    return check(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
}

int qmlp_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, qmlp_hip_stream stream)
{
    if (bytes == 0) return 0;
    if (int rc = check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost,
                                      static_cast<hipStream_t>(stream)), "hipMemcpyAsync(D2H)")) return rc;
    return check(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
}

int qmlp_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, qmlp_hip_stream stream)
{
    if (bytes == 0) return 0;
    return check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice,
                                static_cast<hipStream_t>(stream)), "hipMemcpyAsync(D2D)");
}

int qmlp_hip_device_synchronize(void) { return check(hipDeviceSynchronize(), "hipDeviceSynchronize"); }

int qmlp_hip_stream_create(qmlp_hip_stream* stream)
{
    hipStream_t s;
    if (int rc = check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags")) return rc;
    *stream = s;
    return 0;
}

int qmlp_hip_stream_destroy(qmlp_hip_stream stream)
{
    if (!stream) return 0;
    return check(hipStreamDestroy(static_cast<hipStream_t>(stream)), "hipStreamDestroy");
}

int qmlp_hip_stream_synchronize(qmlp_hip_stream stream)
{
    return check(hipStreamSynchronize(static_cast<hipStream_t>(stream)), "hipStreamSynchronize");
}

int qmlp_hip_event_create(qmlp_hip_event* event, int enable_timing)
{
    hipEvent_t e;
    if (int rc = check(hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming),
                       "hipEventCreateWithFlags")) return rc;
    *event = e;
    return 0;
}

int qmlp_hip_event_destroy(qmlp_hip_event event)
{
    if (!event) return 0;
    return check(hipEventDestroy(static_cast<hipEvent_t>(event)), "hipEventDestroy");
}

int qmlp_hip_event_record(qmlp_hip_event event, qmlp_hip_stream stream)
{
    return check(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)), "hipEventRecord");
}

int qmlp_hip_event_synchronize(qmlp_hip_event event)
{
    return check(hipEventSynchronize(static_cast<hipEvent_t>(event)), "hipEventSynchronize");
}

int qmlp_hip_stream_wait_event(qmlp_hip_stream stream, qmlp_hip_event event)
{
    return check(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0),
                 "hipStreamWaitEvent");
}

int qmlp_hip_event_elapsed_ms(qmlp_hip_event start, qmlp_hip_event stop, float* ms)
{
    return check(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)),
                 "hipEventElapsedTime");
}

static std::string resolveArchitecture(const char* arch)
{
    if (arch && *arch) return arch;
    std::string archName;
    int count = 0;
    qmlp_hip_device_count(&count);
    if (count > 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess)
            archName = p.gcnArchName;
    }
    if (archName.empty()) archName = "gfx950";
    return archName;
}

int qmlp_hip_compile_target(const char* arch, char** target)
{
    if (!target) return fail("qmlp_hip_compile_target: target is NULL");
    int major = 0, minor = 0;
    if (int rc = checkRtc(hiprtcVersion(&major, &minor), "hiprtcVersion")) return rc;
    // the processor without its feature suffixes (":sramecc+:xnack-"): a code object compiled for the plain
    // name runs with any of them, and a cache filled on a machine without a GPU has to be found on one with
    std::string processor = resolveArchitecture(arch);
    processor = processor.substr(0, processor.find(':'));
    const std::string text = processor + ";hiprtc " + std::to_string(major) + "." + std::to_string(minor);
    *target = static_cast<char*>(std::malloc(text.size() + 1));
    if (!*target) return fail("qmlp_hip_compile_target: out of memory");
    std::memcpy(*target, text.c_str(), text.size() + 1);
    return 0;
}

int qmlp_hip_module_compile(const char* source, const char* source_name,
                            const char* const* header_names, const char* const* headers,
                            int num_headers,
                            const char* const* name_expressions, int num_expressions,
                            const char* const* options, int num_options,
                            const char* arch,
                            qmlp_hip_module* module, char** log)
{
    *module = nullptr;
    if (log) *log = nullptr;

    const std::string archName = resolveArchitecture(arch);

    hiprtcProgram prog;
    if (int rc = checkRtc(hiprtcCreateProgram(&prog, source, source_name ? source_name : "qmlp_kernel.hip",
                                              num_headers, const_cast<const char**>(headers),
                                              const_cast<const char**>(header_names)),
                          "hiprtcCreateProgram")) return rc;
    for (int i = 0; i < num_expressions; ++i) {
        if (int rc = checkRtc(hiprtcAddNameExpression(prog, name_expressions[i]), "hiprtcAddNameExpression")) {
            hiprtcDestroyProgram(&prog);
            return rc;
        }
    }
    std::vector<std::string> optStorage;
    optStorage.push_back("--offload-arch=" + archName);
    for (int i = 0; i < num_options; ++i) optStorage.emplace_back(options[i]);
    std::vector<const char*> opts;
    for (auto& o : optStorage) opts.push_back(o.c_str());

    hiprtcResult res = hiprtcCompileProgram(prog, static_cast<int>(opts.size()), opts.data());
    std::string logText;
    size_t logSize = 0;
    if (hiprtcGetProgramLogSize(prog, &logSize) == HIPRTC_SUCCESS && logSize > 1) {
        logText.resize(logSize);
        hiprtcGetProgramLog(prog, &logText[0]);
        while (!logText.empty() && logText.back() == '\0') logText.pop_back();
    }
    if (log && !logText.empty()) {
        *log = static_cast<char*>(std::malloc(logText.size() + 1));
        std::memcpy(*log, logText.c_str(), logText.size() + 1);
    }
    if (res != HIPRTC_SUCCESS) {
        int rc = checkRtc(res, "hiprtcCompileProgram", logText);
        hiprtcDestroyProgram(&prog);
        return rc;
    }

    auto* m = new qmlp_hip_module_s();
    for (int i = 0; i < num_expressions; ++i) {
        const char* lowered = nullptr;
        if (int rc = checkRtc(hiprtcGetLoweredName(prog, name_expressions[i], &lowered), "hiprtcGetLoweredName")) {
            hiprtcDestroyProgram(&prog);
            delete m;
            return rc;
        }
        m->lowered[name_expressions[i]] = lowered;
    }
    size_t codeSize = 0;
    if (int rc = checkRtc(hiprtcGetCodeSize(prog, &codeSize), "hiprtcGetCodeSize")) {
        hiprtcDestroyProgram(&prog);
        delete m;
        return rc;
    }
    m->code.resize(codeSize);
    if (int rc = checkRtc(hiprtcGetCode(prog, m->code.data()), "hiprtcGetCode")) {
        hiprtcDestroyProgram(&prog);
        delete m;
        return rc;
    }
    hiprtcDestroyProgram(&prog);
    *module = m;
    return 0;
}

void qmlp_hip_free_string(char* s) { std::free(s); }

int qmlp_hip_module_from_code(const void* code, size_t size, qmlp_hip_module* module)
{
    auto* m = new qmlp_hip_module_s();
    m->code.assign(static_cast<const char*>(code), static_cast<const char*>(code) + size);
    *module = m;
    return 0;
}

int qmlp_hip_module_code(qmlp_hip_module module, const void** code, size_t* size)
{
    *code = module->code.data();
    *size = module->code.size();
    return 0;
}

int qmlp_hip_module_lowered_name(qmlp_hip_module module, const char* name_expression, const char** lowered)
{
    auto it = module->lowered.find(name_expression);
    if (it == module->lowered.end())
        return fail(std::string("no lowered name recorded for '") + name_expression + "'");
    *lowered = it->second.c_str();
    return 0;
}

int qmlp_hip_module_load(qmlp_hip_module module)
{
    std::lock_guard<std::mutex> lock(module->mutex);
    if (module->loaded) return 0;
    if (int rc = check(hipModuleLoadData(&module->module, module->code.data()), "hipModuleLoadData")) return rc;
    module->loaded = true;
    return 0;
}

int qmlp_hip_module_destroy(qmlp_hip_module module)
{
    if (!module) return 0;
    int rc = 0;
    for (auto& kv : module->functions) delete kv.second;
    if (module->loaded) rc = check(hipModuleUnload(module->module), "hipModuleUnload");
    delete module;
    return rc;
}

int qmlp_hip_module_get_function(qmlp_hip_module module, const char* lowered_name, qmlp_hip_function* function)
{
    if (int rc = qmlp_hip_module_load(module)) return rc;
    std::lock_guard<std::mutex> lock(module->mutex);
    auto it = module->functions.find(lowered_name);
    if (it != module->functions.end()) {
        *function = it->second;
        return 0;
    }
    hipFunction_t fn;
    if (int rc = check(hipModuleGetFunction(&fn, module->module, lowered_name), "hipModuleGetFunction")) return rc;
    auto* f = new qmlp_hip_function_s();
    f->fn = fn;
    f->name = lowered_name;
    module->functions[lowered_name] = f;
    *function = f;
    return 0;
}

int qmlp_hip_module_get_global(qmlp_hip_module module, const char* name, void** device_ptr, size_t* bytes)
{
    if (int rc = qmlp_hip_module_load(module)) return rc;
    hipDeviceptr_t p;
    size_t n = 0;
    if (int rc = check(hipModuleGetGlobal(&p, &n, module->module, name), "hipModuleGetGlobal")) return rc;
    *device_ptr = p;
    if (bytes) *bytes = n;
    return 0;
}

int qmlp_hip_function_occupancy(qmlp_hip_function function, size_t dynamic_lds_bytes,
                                int block_size_limit, int* block_size, int* min_grid_size)
{
    int grid = 0, block = 0;
    if (int rc = check(hipModuleOccupancyMaxPotentialBlockSize(&grid, &block, function->fn, dynamic_lds_bytes,
                                                               block_size_limit),
                       "hipModuleOccupancyMaxPotentialBlockSize")) return rc;
    *block_size = block;
    *min_grid_size = grid;
    return 0;
}

int qmlp_hip_function_blocks_per_cu(qmlp_hip_function function, int block_size, size_t dynamic_lds_bytes,
                                    int* blocks_per_cu)
{
    int blocks = 0;
    if (int rc = check(hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, function->fn, block_size,
                                                                          dynamic_lds_bytes),
                       "hipModuleOccupancyMaxActiveBlocksPerMultiprocessor")) return rc;
    *blocks_per_cu = blocks;
    return 0;
}

int qmlp_hip_function_attributes(qmlp_hip_function function, int* num_vgprs, int* static_lds_bytes,
                                 int* max_threads_per_block, int* scratch_bytes)
{
    int v = 0;
    if (num_vgprs) {
        if (int rc = check(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, function->fn), "hipFuncGetAttribute")) return rc;
        *num_vgprs = v;
    }
    if (static_lds_bytes) {
        if (int rc = check(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, function->fn), "hipFuncGetAttribute")) return rc;
        *static_lds_bytes = v;
    }
    if (max_threads_per_block) {
        if (int rc = check(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, function->fn), "hipFuncGetAttribute")) return rc;
        *max_threads_per_block = v;
    }
    if (scratch_bytes) {
        if (int rc = check(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, function->fn), "hipFuncGetAttribute")) return rc;
        *scratch_bytes = v;
    }
    return 0;
}

int qmlp_hip_launch(qmlp_hip_function function, unsigned grid_x, unsigned block_x,
                    unsigned dynamic_lds_bytes, qmlp_hip_stream stream, void** args)
{
    if (grid_x == 0) return 0;
    return check(hipModuleLaunchKernel(function->fn, grid_x, 1, 1, block_x, 1, 1, dynamic_lds_bytes,
                                       static_cast<hipStream_t>(stream), args, nullptr),
                 "hipModuleLaunchKernel");
}

} // extern "C"
