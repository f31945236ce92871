#include <qmlp/qmlp.h>

#include <cstdlib>
#include <dlfcn.h>

QUICKMLP_NAMESPACE_BEGIN

std::filesystem::path QuickMLP::LocateKernelDirectory()
{
    namespace fs = std::filesystem;
    std::error_code ec;
    if (const char* env = std::getenv("QMLP_KERNEL_DIR")) {
        if (fs::is_directory(fs::path(env) / "qmlp" / "kernels", ec)) return env;
    }
    // relative to the shared library this function lives in
    Dl_info info;
    if (dladdr(reinterpret_cast<void*>(&QuickMLP::LocateKernelDirectory), &info) && info.dli_fname) {
        fs::path lib = fs::absolute(info.dli_fname, ec).parent_path();
        for (const fs::path& cand : {lib / "kernels", lib / ".." / "csrc" / "kernels", lib / "csrc" / "kernels"}) {
            if (fs::is_directory(cand / "qmlp" / "kernels", ec)) return fs::weakly_canonical(cand, ec);
        }
    }
    // relative to this source file (in-tree builds)
    fs::path src(__FILE__);
    fs::path cand = src.parent_path().parent_path() / "kernels";
    if (fs::is_directory(cand / "qmlp" / "kernels", ec)) return cand;
    throw configuration_error("Cannot locate the QuickMLP kernel sources; set QMLP_KERNEL_DIR");
}

QuickMLP::QuickMLP()
    : logger_(std::make_shared<Logger>("qmlp"))
    , kl_(std::make_shared<KernelLoader>(logger_))
    , enableCompileDebugMode_(false)
{
    if (const char* lvl = std::getenv("QMLP_LOG_LEVEL")) {
        try { setLogLevel(std::string(lvl)); } catch (...) {}
    }
    kl_->setCacheDir(KernelLoader::DEFAULT_CACHE_DIR);
    kl_->setKernelDirectory(LocateKernelDirectory());
}

std::unique_ptr<QuickMLP> QuickMLP::INSTANCE = {};

QuickMLP& QuickMLP::Instance()
{
    if (!INSTANCE) INSTANCE = std::unique_ptr<QuickMLP>(new QuickMLP);
    return *INSTANCE;
}

void QuickMLP::DeleteInstance() { INSTANCE = {}; }

bool QuickMLP::isHipAvailable() const { return kl_->isHipAvailable(); }

void QuickMLP::checkHipAvailable() const { kl_->checkHipAvailable(); }

logger_t QuickMLP::getLogger() const { return logger_; }

void QuickMLP::setLogLevel(Logger::Level level) { logger_->set_level(level); }

void QuickMLP::setLogLevel(const std::string& levelName)
{
    Logger::Level level;
    if (levelName == "off") level = Logger::OFF;
    else if (levelName == "debug") level = Logger::DEBUG;
    else if (levelName == "info") level = Logger::INFO;
    else if (levelName == "warn") level = Logger::WARN;
    else if (levelName == "error") level = Logger::ERROR;
    else
        throw std::runtime_error("Unknown log level name '" + levelName
                                 + "', only 'off', 'debug', 'info', 'warn', 'error' are recognized");
    setLogLevel(level);
}

KernelLoader_ptr QuickMLP::kernelLoader() const { return kl_; }

void QuickMLP::setCompileDebugMode(bool enable) { enableCompileDebugMode_ = enable; }

int QuickMLP::getCompileFlags() const
{
    int compileFlags = KernelLoader::CompileThrowOnError;
    if (enableCompileDebugMode_) compileFlags |= KernelLoader::CompileDebugMode;
    return compileFlags;
}

QUICKMLP_NAMESPACE_END
