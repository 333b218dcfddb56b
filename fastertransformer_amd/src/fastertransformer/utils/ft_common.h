// Error handling, logging and string helpers of the host layer code.
// Mirrors the contract of the reference's src/fastertransformer/utils/cuda_utils.h:115-217
// (check_cuda_error / FT_CHECK / FT_CHECK_WITH_INFO throw std::runtime_error),
// utils/string_utils.h (fmtstr, vec2str) and utils/logger.h:93-104 (FT_LOG_* macros,
// level from the FT_LOG_LEVEL environment variable).
#pragma once
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "ftk_sampling.h"

namespace fastertransformer {

inline std::string fmtstr(const char* format, ...)
{
    va_list args;
    va_start(args, format);
    va_list copy;
    va_copy(copy, args);
    const int n = std::vsnprintf(nullptr, 0, format, copy);
    va_end(copy);
    std::string out(n > 0 ? (size_t)n : 0, '\0');
    if (n > 0) {
        std::vsnprintf(&out[0], (size_t)n + 1, format, args);
    }
    va_end(args);
    return out;
}

template<typename V>
inline std::string vec2str(const std::vector<V>& v)
{
    std::ostringstream ss;
    ss << "(";
    for (size_t i = 0; i < v.size(); ++i) {
        ss << (i ? ", " : "") << v[i];
    }
    ss << ")";
    return ss.str();
}

class Logger {
public:
    enum Level { TRACE = 0, DEBUG = 10, INFO = 20, WARNING = 30, ERROR = 40 };
    static Logger& getLogger()
    {
        static Logger instance;
        return instance;
    }
    Level level() const
    {
        return level_;
    }
    void log(Level lvl, const char* tag, const std::string& msg) const
    {
        if (lvl >= level_) {
            std::fprintf(lvl >= WARNING ? stderr : stdout, "[FT][%s] %s\n", tag, msg.c_str());
        }
    }

private:
    Logger()
    {
        const char* env = std::getenv("FT_LOG_LEVEL");
        level_          = WARNING;
        if (env != nullptr) {
            const std::string s(env);
            level_ = s == "TRACE" ? TRACE : s == "DEBUG" ? DEBUG : s == "INFO" ? INFO : s == "ERROR" ? ERROR : WARNING;
        }
    }
    Level level_;
};

#define FT_LOG(lvl, tag, ...)                                                                                          \
    do {                                                                                                               \
        if (::fastertransformer::Logger::lvl >= ::fastertransformer::Logger::getLogger().level()) {                    \
            ::fastertransformer::Logger::getLogger().log(::fastertransformer::Logger::lvl, tag,                        \
                                                         ::fastertransformer::fmtstr(__VA_ARGS__));                    \
        }                                                                                                              \
    } while (0)
#define FT_LOG_TRACE(...) FT_LOG(TRACE, "TRACE", __VA_ARGS__)
#define FT_LOG_DEBUG(...) FT_LOG(DEBUG, "DEBUG", __VA_ARGS__)
#define FT_LOG_INFO(...) FT_LOG(INFO, "INFO", __VA_ARGS__)
#define FT_LOG_WARNING(...) FT_LOG(WARNING, "WARNING", __VA_ARGS__)
#define FT_LOG_ERROR(...) FT_LOG(ERROR, "ERROR", __VA_ARGS__)

[[noreturn]] inline void throwRuntimeError(const char* file, int line, const std::string& info)
{
    throw std::runtime_error(std::string("[FT][ERROR] ") + info + " Assertion fail: " + file + ":"
                             + std::to_string(line) + " \n");
}

#define FT_CHECK(val)                                                                                                  \
    do {                                                                                                               \
        if (!(val)) {                                                                                                  \
            ::fastertransformer::throwRuntimeError(__FILE__, __LINE__, "");                                            \
        }                                                                                                              \
    } while (0)

#define FT_CHECK_WITH_INFO(val, info)                                                                                  \
    do {                                                                                                               \
        if (!(val)) {                                                                                                  \
            ::fastertransformer::throwRuntimeError(__FILE__, __LINE__, (info));                                        \
        }                                                                                                              \
    } while (0)

inline void checkHip(hipError_t e, const char* what, const char* file, int line)
{
    if (e != hipSuccess) {
        throw std::runtime_error(std::string("[FT][ERROR] HIP runtime error: ") + hipGetErrorString(e) + " " + file
                                 + ":" + std::to_string(line) + " '" + what + "'");
    }
}
#define check_hip_error(val) ::fastertransformer::checkHip((val), #val, __FILE__, __LINE__)

// Return codes of the C ABI -> the exception the reference launcher would have thrown.
inline void checkFtk(int code, const char* what, const char* file, int line)
{
    if (code == 0) {
        return;
    }
    if (code == FTK_ERR_TOPK_DOMAIN) {
        throw std::domain_error(std::string("top-k kernel supports 1<=k<=1024 (") + what + ")");
    }
    throw std::runtime_error(std::string("[FT][ERROR] ") + ftk_error_string(code) + " " + file + ":"
                             + std::to_string(line) + " '" + what + "'");
}
#define check_ftk(val) ::fastertransformer::checkFtk((val), #val, __FILE__, __LINE__)

// With FT_DEBUG_LEVEL=DEBUG every launch is followed by a device synchronise + error check
// (the reference's sync_check_cuda_error, utils/cuda_utils.h:127-154).
inline void syncAndCheck(const char* file, int line)
{
    static const bool debug = []() {
        const char* env = std::getenv("FT_DEBUG_LEVEL");
        return env != nullptr && std::string(env) == "DEBUG";
    }();
    if (debug) {
        checkHip(hipDeviceSynchronize(), "hipDeviceSynchronize", file, line);
        checkHip(hipGetLastError(), "hipGetLastError", file, line);
    }
}
#define sync_check_hip_error() ::fastertransformer::syncAndCheck(__FILE__, __LINE__)

}  // namespace fastertransformer
