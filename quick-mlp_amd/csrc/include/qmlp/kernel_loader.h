#pragma once
// Runtime kernel loader: turns generated source text into launchable gfx950 kernels
// through the C ABI in qmlp_hip.h (hipRTC + HIP module API), with an on-disk cache
// of compiled code objects. Takes the place of the external CUDA/NVRTC kernel loader
// the reference is built on (API reconstructed from its call sites, e.g.
// src_cpp/src/fused_network.cpp:397,465-485 and src_cpp/src/qmlp.cpp:10-22).

#include "common.h"
#include "errors.h"
#include "logger.h"

#include <filesystem>
#include <map>
#include <memory>
#include <mutex>
#include <optional>
#include <string>
#include <vector>

struct qmlp_hip_module_s;
struct qmlp_hip_function_s;

QUICKMLP_NAMESPACE_BEGIN

class KernelLoader;

/** A compiled, loaded __global__ function. Cheap to copy. */
class KernelFunction
{
    friend class KernelLoader;
    std::shared_ptr<qmlp_hip_module_s> module_;
    qmlp_hip_function_s* function_ = nullptr;
    std::string name_;
    mutable int bestBlockSize_ = 0;
    mutable int minGridSize_ = 0;

    void queryOccupancy() const;

public:
    KernelFunction() = default;

    [[nodiscard]] bool defined() const { return function_ != nullptr; }
    [[nodiscard]] const std::string& name() const { return name_; }

    /** Block size that maximizes occupancy (no dynamic LDS assumed). */
    [[nodiscard]] int bestBlockSize() const;
    /** Grid size that fills the device once at bestBlockSize(). */
    [[nodiscard]] int minGridSize() const;
    /** Blocks of 'blockSize' threads with 'dynamicLdsBytes' that fill the device once. */
    [[nodiscard]] int fullGridSize(int blockSize, size_t dynamicLdsBytes) const;
    /** Compute units of the device. */
    [[nodiscard]] static int computeUnits();
    [[nodiscard]] int numVgprs() const;
    [[nodiscard]] int scratchBytes() const;

    /** Launches with an array of pointers to the arguments (one per kernel parameter). */
    void launch(unsigned gridSize, unsigned blockSize, unsigned dynamicLdsBytes, stream_t stream, void** args) const;

    /** Launches with the arguments passed by value. */
    template <typename... Args>
    void call(unsigned gridSize, unsigned blockSize, unsigned dynamicLdsBytes, stream_t stream, Args... args) const
    {
        void* ptrs[] = {static_cast<void*>(&args)...};
        launch(gridSize, blockSize, dynamicLdsBytes, stream, ptrs);
    }
};

class KernelLoader
{
public:
    enum CompilationFlags
    {
        CompileDebugMode = 1,      // -g, reduced optimization
        CompileThrowOnError = 2,   // throw instead of returning an empty optional
        CompileOnly = 4,           // compile (and cache) without loading onto a device
        CompileOffline = 8         // with the offline compiler of the installed ROCm where there is one (see hasOfflineCompiler)
    };
    static const std::filesystem::path DEFAULT_CACHE_DIR;

    explicit KernelLoader(logger_t logger);
    ~KernelLoader();

    /** Directory for compiled code objects; empty disables the disk cache. */
    void setCacheDir(const std::filesystem::path& dir);
    void disableCache();
    /** Root directory of the device sources (contains qmlp/kernels/...). */
    void setKernelDirectory(const std::filesystem::path& dir);
    [[nodiscard]] const std::filesystem::path& kernelDirectory() const { return kernelDir_; }

    /** Content of a file below the kernel directory, e.g. "qmlp/kernels/network_forward.h". */
    [[nodiscard]] std::optional<std::string> findFile(const std::string& name) const;
    /** The include line for a device header. */
    [[nodiscard]] static std::string MainFile(const std::string& name);

    [[nodiscard]] bool isHipAvailable() const;
    void checkHipAvailable() const;

    /**
     * Compiles 'source' (or fetches it from the caches) and returns the function with
     * the C++ name 'kernelName' (template arguments allowed).
     * With CompileOnly the returned function is undefined but the code object is cached.
     * offlineOptions: further options for the offline compiler where CompileOffline takes effect (the run-time
     * compiler, which may not know them, never sees them).
     */
    std::optional<KernelFunction> getKernel(const std::string& kernelName, const std::string& source, int flags,
                                            const std::vector<std::string>& offlineOptions = {});

    /**
     * True if kernels can be compiled by the offline compiler of the installed ROCm (`<ROCM_PATH>/bin/hipcc`, run as
     * a child process) instead of the run-time compiler of the process. The run-time compiler is whatever
     * `libhiprtc` the process has loaded: a Python process that imported torch first compiles with the one that torch
     * ships, which can be older than the installed ROCm (register allocation of kernels that hold many matrix-core
     * accumulators differs a lot between them). `QMLP_COMPILER=hiprtc` in the environment switches it off. Only
     * kernels without template arguments can take this path (their symbol is found by its mangled qualified name);
     * a failure of the child process falls back to the run-time compiler.
     */
    [[nodiscard]] static bool hasOfflineCompiler();

    /** Drops all in-memory modules (kernels already handed out stay valid). */
    void clearMemoryCache();

    /** Statistics for tests and logs. */
    [[nodiscard]] int numCompilations() const { return numCompilations_; }
    [[nodiscard]] int numDiskHits() const { return numDiskHits_; }
    [[nodiscard]] int numOfflineCompilations() const { return numOfflineCompilations_; }

private:
    struct Entry
    {
        std::shared_ptr<qmlp_hip_module_s> module;
        std::map<std::string, std::string> lowered;
    };

    logger_t logger_;
    std::filesystem::path cacheDir_;
    std::filesystem::path kernelDir_;
    std::vector<std::string> headerNames_;
    std::vector<std::string> headerContents_;
    std::map<std::string, Entry> modules_;   // key -> module
    std::mutex mutex_;
    int numCompilations_ = 0;
    int numDiskHits_ = 0;
    int numOfflineCompilations_ = 0;

    void loadHeaders();
    /** Digest of the device headers that 'source' includes, directly or through other headers. */
    std::string includedHeadersDigest(const std::string& source) const;
    std::string cacheKey(const std::string& kernelName, const std::string& source,
                         const std::vector<std::string>& options) const;
    bool loadFromDisk(const std::string& key, Entry& entry);
    void saveToDisk(const std::string& key, const Entry& entry);
    /** The code object of `source` from the offline compiler and the symbol of the kernel in it; false (with the reason in `log`) if anything fails. */
    bool compileOffline(const std::string& kernelName, const std::string& source, const std::vector<std::string>& options,
                        Entry& entry, std::string& log) const;
};
typedef std::shared_ptr<KernelLoader> KernelLoader_ptr;

QUICKMLP_NAMESPACE_END
