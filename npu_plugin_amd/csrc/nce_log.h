// The log object behind nce_log_handle_t, shared by the host-side translation units.
#pragma once

#include <cstdarg>
#include <cstdio>
#include <mutex>
#include <string>

struct nce_log_s {
    std::mutex mu;
    std::string text;
    int level = 1;

    void add(int lvl, const char* fmt, ...) {
        if (lvl > level) return;
        char buf[1024];
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(buf, sizeof(buf), fmt, ap);
        va_end(ap);
        std::lock_guard<std::mutex> lk(mu);
        if (text.size() > (1u << 20)) text.clear();  // bounded
        text += buf;
        text += '\n';
    }
};
