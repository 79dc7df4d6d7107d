// Host-side tracing of the engine: named ranges for rocprofv3's marker trace and the executor log.
//
// Ranges: the ROCTx entry points are looked up in librocprofiler-sdk-roctx at first use, so the
// engine carries no link-time dependency on the profiler; without the library a range costs one
// branch.  Under `rocprofv3 --marker-trace` every range shows up with its host start / end time
// next to the kernels and copies it caused.
//
// Log: the reference writes log_executor_<gpu>.txt through spdlog at the level EXECUTOR_LOG_LEVEL
// names (cuda_server.hpp:56-71; sections timed there: CheckMalloc memory_manager.hpp:499-501,
// Transfer 425-431, Evict 258, request completion cuda_server.hpp:294-295).  Same variable and
// level names here; one difference: a library stays silent unless asked, so the default is "off",
// and the file goes to TORPOR_LOG_DIR (default: the working directory).
#pragma once
#include <dlfcn.h>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <mutex>
#include <string>

namespace tp {

class Roctx {
public:
    static Roctx& get() {
        static Roctx r;
        return r;
    }
    void push(const char* name) {
        if (push_) push_(name);
    }
    void pop() {
        if (pop_) pop_();
    }
    // A range that may be closed by another call, or on another thread, than the one that opened it.
    uint64_t start(const char* name) { return start_ ? start_(name) : 0; }
    void stop(uint64_t id) {
        if (stop_ && id) stop_(id);
    }
    bool available() const { return push_ != nullptr; }

private:
    Roctx() {
        const char* off = std::getenv("TORPOR_ROCTX");
        if (off && off[0] == '0') return;
        void* h = dlopen("librocprofiler-sdk-roctx.so.1", RTLD_NOW | RTLD_LOCAL);
        if (!h) h = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_LOCAL);
        if (!h) return;
        auto p = reinterpret_cast<int (*)(const char*)>(dlsym(h, "roctxRangePushA"));
        auto q = reinterpret_cast<int (*)()>(dlsym(h, "roctxRangePop"));
        if (p && q) {
            push_ = p;
            pop_ = q;
        }
        auto a = reinterpret_cast<uint64_t (*)(const char*)>(dlsym(h, "roctxRangeStartA"));
        auto b = reinterpret_cast<void (*)(uint64_t)>(dlsym(h, "roctxRangeStop"));
        if (a && b) {
            start_ = a;
            stop_ = b;
        }
    }
    uint64_t (*start_)(const char*) = nullptr;
    void (*stop_)(uint64_t) = nullptr;
    int (*push_)(const char*) = nullptr;
    int (*pop_)() = nullptr;
};

// A named range on the calling thread, closed when the object goes out of scope.
class TraceRange {
public:
    TraceRange(const char* what, int id) {
        Roctx& r = Roctx::get();
        if (!r.available()) return;
        char buf[64];
        std::snprintf(buf, sizeof buf, "%s %d", what, id);
        r.push(buf);
        open_ = true;
    }
    ~TraceRange() {
        if (open_) Roctx::get().pop();
    }
    TraceRange(const TraceRange&) = delete;
    TraceRange& operator=(const TraceRange&) = delete;

private:
    bool open_ = false;
};

class ExecLog {
public:
    enum Level : int { DEBUG = 0, INFO = 1, WARN = 2, ERR = 3, OFF = 4 };

    ~ExecLog() { close(); }

    // Level from EXECUTOR_LOG_LEVEL (debug | info | warn | err | off); anything else, or unset: off.
    void open(int device) {
        close();
        const char* lv = std::getenv("EXECUTOR_LOG_LEVEL");
        level_ = OFF;
        if (lv) {
            if (!std::strcmp(lv, "debug")) level_ = DEBUG;
            else if (!std::strcmp(lv, "info")) level_ = INFO;
            else if (!std::strcmp(lv, "warn")) level_ = WARN;
            else if (!std::strcmp(lv, "err")) level_ = ERR;
        }
        if (level_ == OFF) return;
        const char* dir = std::getenv("TORPOR_LOG_DIR");
        std::string path = std::string(dir && *dir ? dir : ".") + "/log_executor_" + std::to_string(device) + ".txt";
        fp_ = std::fopen(path.c_str(), "a");
        if (!fp_) level_ = OFF;
    }
    void close() {
        std::lock_guard<std::mutex> lk(mu_);
        if (fp_) std::fclose(fp_);
        fp_ = nullptr;
        level_ = OFF;
    }
    bool on(int level) const { return level >= level_ && level_ != OFF; }

    void write(int level, const char* fmt, ...) __attribute__((format(printf, 3, 4))) {
        if (!on(level)) return;
        static const char* const names[4] = {"debug", "info", "warning", "error"};
        const auto now = std::chrono::system_clock::now();
        const std::time_t t = std::chrono::system_clock::to_time_t(now);
        const long us = (long)(std::chrono::duration_cast<std::chrono::microseconds>(now.time_since_epoch()).count() % 1000000);
        std::tm tm{};
        localtime_r(&t, &tm);
        char stamp[32];
        std::strftime(stamp, sizeof stamp, "%Y-%m-%d %H:%M:%S", &tm);
        std::lock_guard<std::mutex> lk(mu_);
        if (!fp_) return;
        std::fprintf(fp_, "[%s.%06ld] [%s] ", stamp, us, names[level < 0 ? 0 : (level > 3 ? 3 : level)]);
        va_list ap;
        va_start(ap, fmt);
        std::vfprintf(fp_, fmt, ap);
        va_end(ap);
        std::fputc('\n', fp_);
        if (level >= INFO) std::fflush(fp_);  // flush_on(info), as the reference sets it
    }

private:
    std::mutex mu_;
    FILE* fp_ = nullptr;
    int level_ = OFF;
};

}  // namespace tp
