#include <qmlp/kernel_loader.h>

#include "qmlp_hip.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <unistd.h>

QUICKMLP_NAMESPACE_BEGIN

namespace {

struct ModuleDeleter
{
    void operator()(qmlp_hip_module_s* m) const { qmlp_hip_module_destroy(m); }
};

// 2 x 64-bit FNV-1a with different offsets: a 128-bit content key for the cache
std::string digest(const std::string& data)
{
    uint64_t h1 = 1469598103934665603ull, h2 = 0x9ae16a3b2f90404full;
    for (unsigned char c : data) {
        h1 = (h1 ^ c) * 1099511628211ull;
        h2 = (h2 ^ (c + 0x5bu)) * 0x100000001b3ull;
        h2 ^= h2 >> 29;
    }
    char buf[40];
    std::snprintf(buf, sizeof(buf), "%016llx%016llx", static_cast<unsigned long long>(h1),
                  static_cast<unsigned long long>(h2));
    return buf;
}

std::string readFile(const std::filesystem::path& p)
{
    std::ifstream in(p, std::ios::binary);
    std::stringstream ss;
    ss << in.rdbuf();
    return ss.str();
}

std::string rocmIncludeDir()
{
    const char* env = std::getenv("ROCM_PATH");
    std::string root = env && *env ? env : "/opt/rocm";
    return root + "/include";
}

const char CACHE_MAGIC[8] = {'Q', 'M', 'L', 'P', 'C', 'O', '0', '1'};

} // namespace

// ---------------------------------------------------------------- KernelFunction

void KernelFunction::queryOccupancy() const
{
    if (bestBlockSize_ > 0) return;
    if (!defined()) throw std::runtime_error("KernelFunction is not defined");
    QMLP_HIP_CALL(qmlp_hip_function_occupancy(function_, 0, 0, &bestBlockSize_, &minGridSize_));
}

int KernelFunction::bestBlockSize() const
{
    queryOccupancy();
    return bestBlockSize_;
}

int KernelFunction::minGridSize() const
{
    queryOccupancy();
    return minGridSize_;
}

int KernelFunction::fullGridSize(int blockSize, size_t dynamicLdsBytes) const
{
    if (!defined()) throw std::runtime_error("KernelFunction is not defined");
    // workgroups that are resident at the same time: per compute unit x compute units
    int perCu = 0;
    QMLP_HIP_CALL(qmlp_hip_function_blocks_per_cu(function_, blockSize, dynamicLdsBytes, &perCu));
    return std::max(perCu, 1) * computeUnits();
}

int KernelFunction::computeUnits()
{
    static const int value = [] {
        qmlp_hip_device_props props;
        QMLP_HIP_CALL(qmlp_hip_get_device_props(0, &props));   // one GPU per process
        return std::max(props.compute_units, 1);
    }();
    return value;
}

int KernelFunction::numVgprs() const
{
    int v = 0;
    QMLP_HIP_CALL(qmlp_hip_function_attributes(function_, &v, nullptr, nullptr, nullptr));
    return v;
}

int KernelFunction::scratchBytes() const
{
    int v = 0;
    QMLP_HIP_CALL(qmlp_hip_function_attributes(function_, nullptr, nullptr, nullptr, &v));
    return v;
}

void KernelFunction::launch(unsigned gridSize, unsigned blockSize, unsigned dynamicLdsBytes, stream_t stream,
                            void** args) const
{
    if (!defined()) throw std::runtime_error("KernelFunction is not defined");
    QMLP_HIP_CALL(qmlp_hip_launch(function_, gridSize, blockSize, dynamicLdsBytes, stream, args));
}

// ---------------------------------------------------------------- KernelLoader

static std::filesystem::path defaultCacheDir()
{
    if (const char* env = std::getenv("QMLP_CACHE_DIR")) return env;
    if (const char* home = std::getenv("HOME")) return std::filesystem::path(home) / ".cache" / "qmlp" / "kernels";
    return std::filesystem::temp_directory_path() / "qmlp-kernels";
}
const std::filesystem::path KernelLoader::DEFAULT_CACHE_DIR = defaultCacheDir();

KernelLoader::KernelLoader(logger_t logger) : logger_(std::move(logger)) {}

KernelLoader::~KernelLoader() = default;

void KernelLoader::setCacheDir(const std::filesystem::path& dir)
{
    std::lock_guard<std::mutex> lock(mutex_);
    cacheDir_ = dir;
}

void KernelLoader::disableCache()
{
    std::lock_guard<std::mutex> lock(mutex_);
    cacheDir_.clear();
}

void KernelLoader::setKernelDirectory(const std::filesystem::path& dir)
{
    std::lock_guard<std::mutex> lock(mutex_);
    kernelDir_ = dir;
    loadHeaders();
}

void KernelLoader::loadHeaders()
{
    headerNames_.clear();
    headerContents_.clear();
    std::error_code ec;
    if (!std::filesystem::is_directory(kernelDir_, ec)) return;
    std::vector<std::filesystem::path> files;
    for (auto it = std::filesystem::recursive_directory_iterator(kernelDir_, ec);
         !ec && it != std::filesystem::recursive_directory_iterator(); it.increment(ec)) {
        if (it->is_regular_file() && it->path().extension() == ".h") files.push_back(it->path());
    }
    std::sort(files.begin(), files.end());
    for (const auto& f : files) {
        headerNames_.push_back(std::filesystem::relative(f, kernelDir_).generic_string());
        headerContents_.push_back(readFile(f));
    }
}

std::optional<std::string> KernelLoader::findFile(const std::string& name) const
{
    std::filesystem::path p = kernelDir_ / name;
    std::error_code ec;
    if (!std::filesystem::is_regular_file(p, ec)) return {};
    return readFile(p);
}

std::string KernelLoader::MainFile(const std::string& name)
{
    return "#include <" + name + ">\n";
}

bool KernelLoader::isHipAvailable() const
{
    int count = 0;
    qmlp_hip_device_count(&count);
    return count > 0;
}

void KernelLoader::checkHipAvailable() const
{
    if (!isHipAvailable()) throw hip_error("No HIP device available");
}

std::string KernelLoader::includedHeadersDigest(const std::string& source) const
{
    // transitive closure of the #include lines that name one of the device headers; a header
    // that the source cannot reach does not enter the key, so editing it keeps the cache
    std::vector<bool> used(headerNames_.size(), false);
    std::vector<size_t> todo;
    auto scan = [&](const std::string& text) {
        size_t pos = 0;
        while ((pos = text.find("#include", pos)) != std::string::npos) {
            pos += 8;
            const size_t eol = std::min(text.find('\n', pos), text.size());
            const size_t b = text.find_first_of("<\"", pos);
            if (b == std::string::npos || b >= eol) continue;
            const size_t e = text.find_first_of(">\"", b + 1);
            if (e == std::string::npos || e >= eol) continue;
            const std::string name = text.substr(b + 1, e - b - 1);
            for (size_t i = 0; i < headerNames_.size(); ++i)
                if (!used[i] && headerNames_[i] == name) {
                    used[i] = true;
                    todo.push_back(i);
                }
        }
    };
    scan(source);
    while (!todo.empty()) {
        const size_t i = todo.back();
        todo.pop_back();
        scan(headerContents_[i]);
    }
    std::string all;
    for (size_t i = 0; i < headerNames_.size(); ++i)   // headerNames_ is sorted
        if (used[i]) {
            all += headerNames_[i];
            all += '\0';
            all += headerContents_[i];
            all += '\0';
        }
    return digest(all);
}

std::string KernelLoader::cacheKey(const std::string& kernelName, const std::string& source,
                                   const std::vector<std::string>& options) const
{
    std::string all = includedHeadersDigest(source);
    all += '\0';
    // what the code object is compiled for and with: a cache directory may outlive a ROCm update or be
    // carried to a machine with another GPU
    {
        char* target = nullptr;
        if (qmlp_hip_compile_target(std::getenv("QMLP_OFFLOAD_ARCH"), &target) == 0 && target) {
            all += target;
            qmlp_hip_free_string(target);
        }
    }
    all += '\0';
    all += kernelName;
    all += '\0';
    for (const auto& o : options) {
        all += o;
        all += '\0';
    }
    all += source;
    return digest(all);
}

bool KernelLoader::loadFromDisk(const std::string& key, Entry& entry)
{
    if (cacheDir_.empty()) return false;
    std::filesystem::path p = cacheDir_ / (key + ".co");
    std::ifstream in(p, std::ios::binary);
    if (!in) return false;
    char magic[8];
    in.read(magic, 8);
    if (!in || std::memcmp(magic, CACHE_MAGIC, 8) != 0) return false;
    auto readU64 = [&](uint64_t& v) { in.read(reinterpret_cast<char*>(&v), 8); return static_cast<bool>(in); };
    auto readStr = [&](std::string& s) {
        uint64_t n;
        if (!readU64(n) || n > (1ull << 30)) return false;
        s.resize(n);
        in.read(&s[0], static_cast<std::streamsize>(n));
        return static_cast<bool>(in);
    };
    uint64_t numNames;
    if (!readU64(numNames) || numNames > 1024) return false;
    std::map<std::string, std::string> lowered;
    for (uint64_t i = 0; i < numNames; ++i) {
        std::string a, b;
        if (!readStr(a) || !readStr(b)) return false;
        lowered[a] = b;
    }
    std::string code;
    if (!readStr(code)) return false;
    qmlp_hip_module m = nullptr;
    if (qmlp_hip_module_from_code(code.data(), code.size(), &m) != 0) return false;
    entry.module = std::shared_ptr<qmlp_hip_module_s>(m, ModuleDeleter());
    entry.lowered = std::move(lowered);
    return true;
}

void KernelLoader::saveToDisk(const std::string& key, const Entry& entry)
{
    if (cacheDir_.empty()) return;
    std::error_code ec;
    std::filesystem::create_directories(cacheDir_, ec);
    if (ec) {
        logger_->warn("cannot create the kernel cache directory %s: %s", cacheDir_.c_str(), ec.message().c_str());
        return;
    }
    const void* code = nullptr;
    size_t size = 0;
    qmlp_hip_module_code(entry.module.get(), &code, &size);
    std::filesystem::path tmp = cacheDir_ / (key + ".tmp" + std::to_string(static_cast<long long>(::getpid())));
    {
        std::ofstream out(tmp, std::ios::binary);
        if (!out) return;
        auto writeU64 = [&](uint64_t v) { out.write(reinterpret_cast<const char*>(&v), 8); };
        out.write(CACHE_MAGIC, 8);
        writeU64(entry.lowered.size());
        for (const auto& kv : entry.lowered) {
            writeU64(kv.first.size());
            out.write(kv.first.data(), static_cast<std::streamsize>(kv.first.size()));
            writeU64(kv.second.size());
            out.write(kv.second.data(), static_cast<std::streamsize>(kv.second.size()));
        }
        writeU64(size);
        out.write(static_cast<const char*>(code), static_cast<std::streamsize>(size));
    }
    std::filesystem::rename(tmp, cacheDir_ / (key + ".co"), ec);   // atomic publish
    if (ec) std::filesystem::remove(tmp, ec);
}

std::optional<KernelFunction> KernelLoader::getKernel(const std::string& kernelName, const std::string& source,
                                                      int flags)
{
    std::lock_guard<std::mutex> lock(mutex_);
    const bool debug = (flags & CompileDebugMode) != 0;
    const bool throwOnError = (flags & CompileThrowOnError) != 0;
    const bool compileOnly = (flags & CompileOnly) != 0;

    std::vector<std::string> options = {
        "-std=c++17",
        debug ? "-O1" : "-O3",
        "-I" + rocmIncludeDir(),
        // packed fp32 arithmetic is kept off for every kernel of this library
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-Wno-unused-value",
    };
    if (debug) options.emplace_back("-g");
    if (const char* extra = std::getenv("QMLP_EXTRA_COMPILE_FLAGS")) {
        std::stringstream ss(extra);
        std::string tok;
        while (ss >> tok) options.push_back(tok);
    }

    try {
        const std::string key = cacheKey(kernelName, source, options);
        auto it = modules_.find(key);
        if (it == modules_.end()) {
            Entry entry;
            if (loadFromDisk(key, entry)) {
                ++numDiskHits_;
                logger_->debug("kernel %s: code object found in the disk cache (%s)", kernelName.c_str(), key.c_str());
            } else {
                logger_->info("compiling kernel %s", kernelName.c_str());
                if (logger_->should_log(Logger::DEBUG)) logger_->debug("source:\n%s", source.c_str());
                std::vector<const char*> hn, hc, opts;
                for (const auto& n : headerNames_) hn.push_back(n.c_str());
                for (const auto& c : headerContents_) hc.push_back(c.c_str());
                for (const auto& o : options) opts.push_back(o.c_str());
                const char* exprs[] = {kernelName.c_str()};
                qmlp_hip_module m = nullptr;
                char* log = nullptr;
                int rc = qmlp_hip_module_compile(source.c_str(), "qmlp_generated.hip", hn.data(), hc.data(),
                                                 static_cast<int>(hn.size()), exprs, 1, opts.data(),
                                                 static_cast<int>(opts.size()), std::getenv("QMLP_OFFLOAD_ARCH"),
                                                 &m, &log);
                std::string logText = log ? log : "";
                qmlp_hip_free_string(log);
                if (rc != 0) {
                    logger_->error("compilation of %s failed:\n%s", kernelName.c_str(), qmlp_hip_last_error());
                    throw hip_error(std::string("Kernel compilation failed for ") + kernelName + ":\n"
                                    + qmlp_hip_last_error());
                }
                if (!logText.empty()) logger_->debug("compiler log of %s:\n%s", kernelName.c_str(), logText.c_str());
                ++numCompilations_;
                entry.module = std::shared_ptr<qmlp_hip_module_s>(m, ModuleDeleter());
                const char* lowered = nullptr;
                QMLP_HIP_CALL(qmlp_hip_module_lowered_name(m, kernelName.c_str(), &lowered));
                entry.lowered[kernelName] = lowered;
                saveToDisk(key, entry);
            }
            it = modules_.emplace(key, std::move(entry)).first;
        }
        KernelFunction fun;
        fun.name_ = kernelName;
        if (compileOnly) return fun;
        auto lit = it->second.lowered.find(kernelName);
        if (lit == it->second.lowered.end()) throw hip_error("cached module lacks the kernel " + kernelName);
        qmlp_hip_function f = nullptr;
        QMLP_HIP_CALL(qmlp_hip_module_get_function(it->second.module.get(), lit->second.c_str(), &f));
        fun.module_ = it->second.module;
        fun.function_ = f;
        return fun;
    } catch (...) {
        if (throwOnError) throw;
        return {};
    }
}

void KernelLoader::clearMemoryCache()
{
    std::lock_guard<std::mutex> lock(mutex_);
    modules_.clear();
}

QUICKMLP_NAMESPACE_END
