// Launch recorder of the host-only trace build (-DFLA_TRACE_LAUNCHES): see fla_launch.h.
// A record is one line of text, `key=value` pairs separated by ';':
//     kernel=<function with template arguments>;grid=x,y,z;block=n;lds=bytes;a0=...;a1.field=...
// Scalars and pointers are written as they are; parameter structs field by field (the overloads
// of trace_describe in fla_trace_structs.h).  The records of a thread are kept until taken with
// fla_trace_take (declared at the bottom; defined in fla_capi.hip).
#pragma once

#include <stdint.h>

#include <sstream>
#include <string>
#include <type_traits>

extern "C" void fla_trace_append(const char *line);
extern "C" void fla_trace_lds_limit(const char *kernel, int bytes);
// name of the kernel's host symbol (demangled where the C++ runtime can); `fallback` when it has none
extern "C" const char *fla_trace_symbol(const void *kernel, const char *fallback);

namespace fla {
namespace trace {

// e.g. "void fla::tri_xyt_z_fast_kernel<__bf16, 128, 128, false, 1>(fla::TriParams)"
template <auto Kern>
const char *kernel_name() {
    // (the fallback, for kernels with internal linkage: "... [Kern = &(anonymous namespace)::some_kernel]")
    static const char *name = fla_trace_symbol(reinterpret_cast<const void *>(Kern), __PRETTY_FUNCTION__);
    return name;
}

inline void note_lds_limit(const char *kernel, int bytes) { fla_trace_lds_limit(kernel, bytes); }

struct Record {
    std::ostringstream os;
    Record(const char *name, unsigned gx, unsigned gy, unsigned gz, unsigned block, size_t lds) {
        os << "kernel=" << name << ";grid=" << gx << "," << gy << "," << gz << ";block=" << block << ";lds=" << lds;
    }
    template <typename V>
    void field(int arg, const char *name, const V &v) {
        os << ";a" << arg;
        if (name && *name) os << "." << name;
        os << "=";
        if constexpr (std::is_pointer_v<V>)
            os << reinterpret_cast<uintptr_t>(v);
        else if constexpr (std::is_floating_point_v<V>)
            os << (double)v;
        else
            os << (long long)v;
    }
    void commit() { fla_trace_append(os.str().c_str()); }
};

// scalars and pointers
template <typename V, typename = std::enable_if_t<std::is_arithmetic_v<V> || std::is_pointer_v<V>>>
inline void trace_describe(Record &r, int arg, const V &v) {
    r.field(arg, "", v);
}

}  // namespace trace
}  // namespace fla
