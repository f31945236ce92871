#include <qmlp/kernel_loader.h>

#include "qmlp_hip.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <fcntl.h>
#include <spawn.h>
#include <sys/wait.h>
#include <unistd.h>

extern char** environ;

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

std::string rocmRoot()
{
    const char* env = std::getenv("ROCM_PATH");
    return env && *env ? env : "/opt/rocm";
}

// The offline compiler of the installed ROCm: its path (empty: none, or switched off) and what identifies its
// version in a cache key, read from a file so that no process has to be started to look a kernel up.
struct OfflineCompiler
{
    std::string path, id;
};
const OfflineCompiler& offlineCompiler()
{
    static const OfflineCompiler compiler = [] {
        OfflineCompiler c;
        const char* choice = std::getenv("QMLP_COMPILER");
        if (choice && std::string(choice) == "hiprtc") return c;
        const std::string path = rocmRoot() + "/bin/hipcc";
        if (::access(path.c_str(), X_OK) != 0) return c;
        std::string version = readFile(rocmRoot() + "/.info/version");
        version = version.substr(0, version.find_first_of("\r\n"));
        if (version.empty()) return c;   // nothing to tell two installations apart by
        c.path = path;
        c.id = "hipcc " + version;
        return c;
    }();
    return compiler;
}

// Symbols of the kernels in a code object (ELF64, little endian): every kernel has a descriptor "<symbol>.kd".
std::vector<std::string> kernelSymbols(const std::string& elf)
{
    std::vector<std::string> symbols;
    auto u16 = [&](size_t at) { uint16_t v = 0; if (at + 2 <= elf.size()) std::memcpy(&v, elf.data() + at, 2); return v; };
    auto u32 = [&](size_t at) { uint32_t v = 0; if (at + 4 <= elf.size()) std::memcpy(&v, elf.data() + at, 4); return v; };
    auto u64 = [&](size_t at) { uint64_t v = 0; if (at + 8 <= elf.size()) std::memcpy(&v, elf.data() + at, 8); return v; };
    if (elf.size() < 64 || std::memcmp(elf.data(), "\177ELF", 4) != 0 || elf[4] != 2 || elf[5] != 1) return symbols;
    const uint64_t shoff = u64(0x28);
    const uint16_t shentsize = u16(0x3A), shnum = u16(0x3C);
    auto section = [&](uint32_t i) { return shoff + static_cast<uint64_t>(i) * shentsize; };
    for (uint32_t i = 0; i < shnum; ++i) {
        const uint64_t sh = section(i);
        if (sh + 64 > elf.size()) return symbols;
        const uint32_t type = u32(sh + 4);
        if (type != 2 && type != 11) continue;   // SHT_SYMTAB, SHT_DYNSYM
        const uint64_t offset = u64(sh + 24), size = u64(sh + 32), entsize = u64(sh + 56);
        const uint32_t link = u32(sh + 40);
        if (link >= shnum || entsize < 24) continue;
        const uint64_t strOffset = u64(section(link) + 24), strSize = u64(section(link) + 32);
        if (strOffset + strSize > elf.size() || offset + size > elf.size()) continue;
        for (uint64_t at = offset; at + entsize <= offset + size; at += entsize) {
            const uint32_t name = u32(at);
            if (name >= strSize) continue;
            const char* text = elf.data() + strOffset + name;
            const size_t length = ::strnlen(text, strSize - name);
            if (length > 3 && std::memcmp(text + length - 3, ".kd", 3) == 0) {
                std::string symbol(text, length - 3);
                if (std::find(symbols.begin(), symbols.end(), symbol) == symbols.end()) symbols.push_back(std::move(symbol));
            }
        }
    }
    return symbols;
}

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
                                                      int flags, const std::vector<std::string>& offlineOptions)
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

    // (part of the key, not of the command line: a cache filled by one compiler is not taken for the other's)
    const bool offline = (flags & CompileOffline) != 0 && hasOfflineCompiler() && kernelName.find('<') == std::string::npos;
    std::vector<std::string> keyOptions = options;
    if (offline) {
        keyOptions.push_back("compiler: " + offlineCompiler().id);
        keyOptions.insert(keyOptions.end(), offlineOptions.begin(), offlineOptions.end());
    }

    try {
        const std::string key = cacheKey(kernelName, source, keyOptions);
        auto it = modules_.find(key);
        if (it == modules_.end()) {
            Entry entry;
            if (loadFromDisk(key, entry)) {
                ++numDiskHits_;
                logger_->debug("kernel %s: code object found in the disk cache (%s)", kernelName.c_str(), key.c_str());
            } else {
                logger_->info("compiling kernel %s", kernelName.c_str());
                if (logger_->should_log(Logger::DEBUG)) logger_->debug("source:\n%s", source.c_str());
                if (const char* dump = std::getenv("QMLP_DUMP_SOURCES")) {
                    // debugging aid: the source and the name of every kernel that is compiled, by cache key
                    std::error_code dumpError;
                    std::filesystem::create_directories(dump, dumpError);
                    std::ofstream(std::filesystem::path(dump) / (key + ".hip"), std::ios::binary) << source;
                    std::ofstream(std::filesystem::path(dump) / (key + ".name"), std::ios::binary) << kernelName;
                }
                bool compiled = false;
                if (offline) {
                    std::string offlineLog;
                    std::vector<std::string> allOptions = options;
                    allOptions.insert(allOptions.end(), offlineOptions.begin(), offlineOptions.end());
                    compiled = compileOffline(kernelName, source, allOptions, entry, offlineLog);
                    if (compiled) {
                        ++numCompilations_;
                        ++numOfflineCompilations_;
                        if (!offlineLog.empty()) logger_->debug("compiler log of %s:\n%s", kernelName.c_str(), offlineLog.c_str());
                        saveToDisk(key, entry);
                    } else {
                        logger_->warn("offline compilation of %s failed, the run-time compiler takes it: %s", kernelName.c_str(), offlineLog.c_str());
                        entry = Entry();
                    }
                }
                const bool fallback = offline && !compiled;   // stays in memory: the key on disk names the offline compiler
                if (!compiled) {
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
                if (!fallback) saveToDisk(key, entry);
                }
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

bool KernelLoader::hasOfflineCompiler()
{
    return !offlineCompiler().path.empty();
}

bool KernelLoader::compileOffline(const std::string& kernelName, const std::string& source, const std::vector<std::string>& options,
                                  Entry& entry, std::string& log) const
{
    namespace fs = std::filesystem;
    const OfflineCompiler& compiler = offlineCompiler();
    if (compiler.path.empty()) { log = "no offline compiler"; return false; }
    if (kernelName.find('<') != std::string::npos) { log = "kernels with template arguments are left to the run-time compiler"; return false; }
    // A preloaded profiler library would be loaded into the compiler's processes as well and set up the device in each
    // of them before they start their own children: no child processes under a profiler.
    if (const char* preload = std::getenv("LD_PRELOAD")) {
        if (std::strstr(preload, "rocprof") || std::strstr(preload, "roctracer")) { log = "a profiler is preloaded into this process"; return false; }
    }
    std::string processor;
    {
        char* target = nullptr;
        if (qmlp_hip_compile_target(std::getenv("QMLP_OFFLOAD_ARCH"), &target) != 0 || !target) { log = "no compile target"; return false; }
        processor = target;
        qmlp_hip_free_string(target);
        processor = processor.substr(0, processor.find(';'));
    }
    std::error_code ec;
    std::string pattern = (fs::temp_directory_path(ec) / "qmlp-offline-XXXXXX").string();
    if (ec || !::mkdtemp(&pattern[0])) { log = "cannot create a temporary directory"; return false; }
    const fs::path dir = pattern;
    struct Cleanup { fs::path dir; ~Cleanup() { std::error_code e; fs::remove_all(dir, e); } } cleanup{dir};
    // the same headers the run-time compiler is given, from memory: what is on disk may have changed since they were read
    for (size_t i = 0; i < headerNames_.size(); ++i) {
        const fs::path file = dir / "include" / headerNames_[i];
        fs::create_directories(file.parent_path(), ec);
        std::ofstream(file, std::ios::binary) << headerContents_[i];
    }
    std::ofstream(dir / "kernel.hip", std::ios::binary) << source;
    const std::string output = (dir / "kernel.co").string(), messages = (dir / "messages.txt").string();
    std::vector<std::string> arguments = {compiler.path, "--genco", "--no-gpu-bundle-output", "--offload-arch=" + processor};
    for (const auto& o : options) arguments.push_back(o);
    arguments.push_back("-I" + (dir / "include").string());
    arguments.push_back("-o");
    arguments.push_back(output);
    arguments.push_back((dir / "kernel.hip").string());
    std::vector<char*> argv;
    for (auto& a : arguments) argv.push_back(&a[0]);
    argv.push_back(nullptr);
    posix_spawn_file_actions_t actions;
    posix_spawn_file_actions_init(&actions);
    posix_spawn_file_actions_addopen(&actions, 0, "/dev/null", O_RDONLY, 0);
    posix_spawn_file_actions_addopen(&actions, 1, messages.c_str(), O_WRONLY | O_CREAT | O_TRUNC, 0600);
    posix_spawn_file_actions_adddup2(&actions, 1, 2);
    pid_t child = 0;
    const int spawned = posix_spawn(&child, compiler.path.c_str(), &actions, nullptr, argv.data(), environ);
    posix_spawn_file_actions_destroy(&actions);
    if (spawned != 0) { log = std::string("cannot start ") + compiler.path + ": " + std::strerror(spawned); return false; }
    int status = 0;
    while (::waitpid(child, &status, 0) < 0) {
        if (errno != EINTR) { log = "waiting for the compiler failed"; return false; }
    }
    log = readFile(messages);
    if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) {
        log = compiler.path + " failed:\n" + log;
        return false;
    }
    const std::string code = readFile(output);
    // The symbol of a function without template arguments starts with its mangled qualified name, the parameter types
    // follow: _ZN <length><component>... E for a name in namespaces, _Z <length><name> for one outside (or the plain name
    // of an extern "C" function). Two overloads of one name are not told apart: left to the run-time compiler.
    std::string prefix, plain;
    {
        std::vector<std::string> components;
        size_t from = 0;
        for (size_t at; (at = kernelName.find("::", from)) != std::string::npos; from = at + 2) components.push_back(kernelName.substr(from, at - from));
        components.push_back(kernelName.substr(from));
        if (components.size() == 1) {
            plain = components[0];
            prefix = "_Z" + std::to_string(plain.size()) + plain;
        } else {
            prefix = "_ZN";
            for (const auto& c : components) prefix += std::to_string(c.size()) + c;
            prefix += "E";
        }
    }
    std::string symbol;
    int matches = 0;
    for (const std::string& candidate : kernelSymbols(code)) {
        if (candidate.compare(0, prefix.size(), prefix) == 0 || (!plain.empty() && candidate == plain)) {
            symbol = candidate;
            ++matches;
        }
    }
    if (matches > 1) symbol.clear();
    if (symbol.empty()) { log = "the code object of the offline compiler has no kernel " + kernelName + "\n" + log; return false; }
    qmlp_hip_module m = nullptr;
    if (qmlp_hip_module_from_code(code.data(), code.size(), &m) != 0) { log = "cannot keep the code object"; return false; }
    entry.module = std::shared_ptr<qmlp_hip_module_s>(m, ModuleDeleter());
    entry.lowered[kernelName] = symbol;
    return true;
}

void KernelLoader::clearMemoryCache()
{
    std::lock_guard<std::mutex> lock(mutex_);
    modules_.clear();
}

QUICKMLP_NAMESPACE_END
