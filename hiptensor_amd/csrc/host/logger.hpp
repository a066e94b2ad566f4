// Process-wide log sink behind the hiptensorLogger* entry points.
// Behaviour follows library/src/logger.cpp:37-188 of the reference: a bit mask selects
// contexts, output goes to a FILE* (stdout by default) and to an optional callback,
// and every line reads "[pid][YYYY-MM-DD HH:MM:SS][hipTensor][context][function] text".
#pragma once
#include <cstdint>
#include <cstdio>
#include <mutex>

#include <hiptensor/hiptensor_types.hpp>

namespace hipta
{
    class Logger
    {
    public:
        enum class Result
        {
            OK,
            BAD_FILE_NAME,
            BAD_STREAM,
            BAD_MASK,
            BAD_LEVEL,
            OPEN_FAILED
        };

        static Logger& get();

        Result setStream(FILE* stream);
        Result openFile(const char* path);
        Result setCallback(hiptensorLoggerCallback_t cb);
        Result setLevel(int level);
        Result setMask(int32_t mask);
        void   setEnabled(bool on);
        int32_t mask() const;

        void emit(int32_t context, const char* func, const char* text);
        void error(const char* func, const char* text) { emit(HIPTENSOR_LOG_LEVEL_ERROR, func, text); }
        void perf(const char* func, const char* text) { emit(HIPTENSOR_LOG_LEVEL_PERF_TRACE, func, text); }
        void heuristics(const char* func, const char* text)
        {
            emit(HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE, func, text);
        }
        void api(const char* func, const char* text) { emit(HIPTENSOR_LOG_LEVEL_API_TRACE, func, text); }
        // printf-style helpers
        void apif(const char* func, const char* fmt, ...) __attribute__((format(printf, 3, 4)));
        void errorf(const char* func, const char* fmt, ...) __attribute__((format(printf, 3, 4)));

        static const char* resultName(Result r);

    private:
        Logger() = default;
        ~Logger();
        mutable std::mutex        mLock;
        bool                      mEnabled  = true;
        bool                      mOwnsFile = false;
        int32_t                   mMask     = 0;
        FILE*                     mOut      = stdout;
        hiptensorLoggerCallback_t mCallback = nullptr;
    };
}
