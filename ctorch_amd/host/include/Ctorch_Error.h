// The reference's two error conventions (include/Ctorch_Error.h): log(ERROR, ...) prints, counts
// and CONTINUES (:353-405); throwException logs and throws std::runtime_error (:510-515).  This
// front-end keeps both entry points with the same names and meaning; the banner, colours and
// 500 ms start-up sleep of the reference are not reproduced.
#ifndef CTORCH_AMD_HOST_ERROR_H
#define CTORCH_AMD_HOST_ERROR_H
#include <atomic>
#include <cstdio>
#include <stdexcept>
#include <string>

#include "Ctools.h"

class Ctorch_Error {
   public:
    static PrintLevel& level() {
        static PrintLevel l = PrintLevel::MINIUM;
        return l;
    }
    static std::atomic<size_t>& errorCount() {
        static std::atomic<size_t> n{0};
        return n;
    }
    static void setPrintLevel(PrintLevel l) { level() = l; }

    static void log(ErrorLevel lvl, ErrorPlatform platform, ErrorType type, const std::string& msg) {
        if (lvl >= ErrorLevel::ERROR) errorCount()++;
        bool show = lvl >= ErrorLevel::INFO || (lvl == ErrorLevel::DEBUG && level() >= PrintLevel::MEDIUM) ||
                    level() == PrintLevel::FULL;
        if (show)
            std::fprintf(stderr, "[%s] [PLATFORM:%d] [TYPE:%d] %s\n", name(lvl), static_cast<int>(platform),
                         static_cast<int>(type), msg.c_str());
    }
    static void trace(ErrorPlatform platform, const std::string& msg) { log(ErrorLevel::TRACE, platform, ErrorType::UNKNOWN, msg); }
    static void info(ErrorPlatform platform, const std::string& msg) { log(ErrorLevel::INFO, platform, ErrorType::UNKNOWN, msg); }
    static void warn(ErrorPlatform platform, ErrorType type, const std::string& msg) { log(ErrorLevel::WARN, platform, type, msg); }
    static void error(ErrorPlatform platform, ErrorType type, const std::string& msg) { log(ErrorLevel::ERROR, platform, type, msg); }
    [[noreturn]] static void throwException(ErrorPlatform platform, ErrorType type, const std::string& msg) {
        log(ErrorLevel::ERROR, platform, type, msg);
        throw std::runtime_error(msg);
    }

   private:
    static const char* name(ErrorLevel l) {
        switch (l) {
            case ErrorLevel::TRACE: return "TRACE";
            case ErrorLevel::DEBUG: return "DEBUG";
            case ErrorLevel::INFO: return "INFO";
            case ErrorLevel::WARN: return "WARN";
            case ErrorLevel::ERROR: return "ERROR";
            case ErrorLevel::FATAL: return "FATAL";
        }
        return "?";
    }
};
#endif
