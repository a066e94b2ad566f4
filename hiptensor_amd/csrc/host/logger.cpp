#include "logger.hpp"

#include <cstdarg>
#include <cstring>
#include <ctime>
#include <unistd.h>

namespace hipta
{
    Logger& Logger::get()
    {
        static Logger* inst = new Logger(); // intentionally never destroyed: usable during exit
        return *inst;
    }

    Logger::~Logger()
    {
        if(mOwnsFile && mOut)
            fclose(mOut);
    }

    Logger::Result Logger::setStream(FILE* stream)
    {
        std::lock_guard<std::mutex> g(mLock);
        if(!stream)
            return Result::BAD_STREAM;
        if(mOwnsFile && mOut)
            fclose(mOut);
        mOwnsFile = false;
        mOut      = stream;
        return Result::OK;
    }

    Logger::Result Logger::openFile(const char* path)
    {
        std::lock_guard<std::mutex> g(mLock);
        if(mOwnsFile && mOut)
            fclose(mOut);
        mOwnsFile = false;
        mOut      = stdout; // fall back to stdout on any failure, like the reference
        if(!path || !*path)
            return Result::BAD_FILE_NAME;
        FILE* f = fopen(path, "w");
        if(!f)
            return Result::OPEN_FAILED;
        mOut      = f;
        mOwnsFile = true;
        return Result::OK;
    }

    Logger::Result Logger::setCallback(hiptensorLoggerCallback_t cb)
    {
        std::lock_guard<std::mutex> g(mLock);
        mCallback = cb;
        return Result::OK;
    }

    Logger::Result Logger::setLevel(int level)
    {
        std::lock_guard<std::mutex> g(mLock);
        // only single-bit levels (or OFF) are accepted
        switch(level)
        {
        case HIPTENSOR_LOG_LEVEL_OFF:
        case HIPTENSOR_LOG_LEVEL_ERROR:
        case HIPTENSOR_LOG_LEVEL_PERF_TRACE:
        case HIPTENSOR_LOG_LEVEL_PERF_HINT:
        case HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE:
        case HIPTENSOR_LOG_LEVEL_API_TRACE: mMask = level; return Result::OK;
        default: return Result::BAD_LEVEL;
        }
    }

    Logger::Result Logger::setMask(int32_t mask)
    {
        std::lock_guard<std::mutex> g(mLock);
        if(mask < 0 || mask > 0x1F)
            return Result::BAD_MASK;
        mMask = mask;
        return Result::OK;
    }

    void Logger::setEnabled(bool on)
    {
        std::lock_guard<std::mutex> g(mLock);
        mEnabled = on;
    }

    int32_t Logger::mask() const
    {
        std::lock_guard<std::mutex> g(mLock);
        return mMask;
    }

    static const char* contextName(int32_t c)
    {
        switch(c)
        {
        case HIPTENSOR_LOG_LEVEL_ERROR: return "Error";
        case HIPTENSOR_LOG_LEVEL_PERF_TRACE: return "Performance";
        case HIPTENSOR_LOG_LEVEL_PERF_HINT: return "Performance Hint";
        case HIPTENSOR_LOG_LEVEL_HEURISTICS_TRACE: return "Heuristics Trace";
        case HIPTENSOR_LOG_LEVEL_API_TRACE: return "API";
        default: return "";
        }
    }

    void Logger::emit(int32_t context, const char* func, const char* text)
    {
        std::lock_guard<std::mutex> g(mLock);
        if(!mEnabled || (context & mMask) == 0)
            return;
        char      stamp[32];
        time_t    now = time(nullptr);
        struct tm tmv;
        localtime_r(&now, &tmv);
        strftime(stamp, sizeof(stamp), "%F %T", &tmv);
        char line[2304];
        snprintf(line,
                 sizeof(line),
                 "[%d][%s][hipTensor][%s][%s] %s\n",
                 (int)getpid(),
                 stamp,
                 contextName(context),
                 func,
                 text);
        if(mCallback)
            mCallback(context, func, line);
        if(mOut)
            fputs(line, mOut);
    }

    void Logger::apif(const char* func, const char* fmt, ...)
    {
        if((mask() & HIPTENSOR_LOG_LEVEL_API_TRACE) == 0)
            return;
        char    buf[2048];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof(buf), fmt, ap);
        va_end(ap);
        api(func, buf);
    }

    void Logger::errorf(const char* func, const char* fmt, ...)
    {
        if((mask() & HIPTENSOR_LOG_LEVEL_ERROR) == 0)
            return;
        char    buf[2048];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof(buf), fmt, ap);
        va_end(ap);
        error(func, buf);
    }

    const char* Logger::resultName(Result r)
    {
        switch(r)
        {
        case Result::OK: return "SUCCESS";
        case Result::BAD_FILE_NAME: return "INVALID_FILE_NAME";
        case Result::BAD_STREAM: return "INVALID_FILE_STREAM";
        case Result::BAD_MASK: return "INVALID_LOG_MASK";
        case Result::BAD_LEVEL: return "INVALID_LOG_LEVEL";
        case Result::OPEN_FAILED: return "FILE_OPEN_FAILED";
        }
        return "STATUS_UNKNOWN";
    }
}
