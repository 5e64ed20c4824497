#include "graph_log.hpp"

#include <atomic>
#include <cctype>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <ctime>
#include <mutex>

namespace mlel::graphlog {
namespace {

const char *const kNames[4] = {"Error", "Warning", "Info", "Debug"};
std::atomic<int> g_level{-1};  // -1: not read yet
std::mutex g_write;

bool same_word(const char *a, const char *b) {
    for (; *a && *b; a++, b++)
        if (std::tolower((unsigned char)*a) != std::tolower((unsigned char)*b)) return false;
    return *a == 0 && *b == 0;
}

int read_level() {
    const char *env = std::getenv("VMEL_GRAPH_SEVERITY");
    if (env != nullptr)
        for (int i = 0; i < 4; i++)
            if (same_word(env, kNames[i])) return i;
    return (int)Severity::Error;
}

}  // namespace

void reload() { g_level.store(read_level()); }

Severity level() {
    int l = g_level.load();
    if (l < 0) {
        l = read_level();
        g_level.store(l);
    }
    return (Severity)l;
}

bool enabled(Severity severity) { return (int)level() >= (int)severity; }

void write(Severity severity, const std::string &message) {
    if (!enabled(severity)) return;
    const auto now = std::chrono::system_clock::now();
    const long ms = (long)(std::chrono::duration_cast<std::chrono::milliseconds>(now.time_since_epoch()).count() % 1000);
    const std::time_t t = std::chrono::system_clock::to_time_t(now);
    std::tm local{};
    localtime_r(&t, &local);
    char stamp[32];
    std::strftime(stamp, sizeof stamp, "%Y-%m-%d %H:%M:%S", &local);
    std::lock_guard<std::mutex> guard(g_write);
    std::fprintf(stdout, "%s,%03ld [Graph][%s] %s\n", stamp, ms, kNames[(int)severity], message.c_str());
    std::fflush(stdout);
}

}  // namespace mlel::graphlog
