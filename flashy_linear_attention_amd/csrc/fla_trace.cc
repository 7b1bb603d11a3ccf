// Storage and C entry points of the launch recorder (host-only trace build, see fla_launch.h):
// the records of the calling thread, taken as one newline-separated text.
#include <stdint.h>
#include <string.h>

#include <cxxabi.h>
#include <dlfcn.h>
#include <stdlib.h>

#include <string>

namespace {
thread_local std::string g_records;
}

extern "C" {

const char *fla_trace_symbol(const void *kernel, const char *fallback) {
    Dl_info info;
    if (!dladdr(kernel, &info) || !info.dli_sname) return fallback;
    int status = 0;
    char *text = abi::__cxa_demangle(info.dli_sname, nullptr, nullptr, &status);
    return status == 0 && text ? text : strdup(info.dli_sname);  // (kept for the life of the process)
}

void fla_trace_append(const char *line) {
    g_records += line;
    g_records += '\n';
}

void fla_trace_lds_limit(const char *kernel, int bytes) {
    g_records += "lds_limit=" + std::to_string(bytes) + ";kernel=" + kernel + "\n";
}

// Copies the records so far (and forgets them) into buf, NUL-terminated; returns the length
// needed including the NUL.  With buf == NULL or too small nothing is forgotten.
int64_t fla_trace_take(char *buf, int64_t capacity) {
    const int64_t need = (int64_t)g_records.size() + 1;
    if (!buf || capacity < need) return need;
    memcpy(buf, g_records.c_str(), (size_t)need);
    g_records.clear();
    return need;
}

}  // extern "C"
