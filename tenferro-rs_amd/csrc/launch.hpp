// launch.hpp -- kernel launch that hands the dispatch the profiling events of the current call, if any.
#pragma once
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <cxxabi.h>

#include <cstdlib>
#include <string>
#include <typeinfo>

#include "internal.hpp"

namespace tfh {
// "(kernel<arguments as instantiated>)" for a kernel function, e.g. "(gemm128_kernel<double, true, false, true, 1, 1, 128>)":
// the name a kernel trace shows, without return type, namespaces and parameter list.  Built once per instantiation
// from the demangled name of a type that carries the kernel's address as its template argument.
template <auto K> struct KernelTag {};
inline std::string kernel_label_from(const char* mangled) {
    int status = 0;
    char* dem = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
    std::string p = dem ? dem : mangled;   // "tfh::KernelTag<&(void tfh::gemm::gemm128_kernel<double, ...>(tfh::gemm::GemmArgs))>"
    std::free(dem);
    for (const char* ns : {"tfh::gemm::", "tfh::(anonymous namespace)::", "(anonymous namespace)::", "tfh::"})
        for (size_t at; (at = p.find(ns)) != std::string::npos;) p.erase(at, std::string(ns).size());
    const size_t a = p.find("&(void ");
    if (a != std::string::npos) p = p.substr(a + 7);
    int depth = 0;
    for (size_t i = 0; i < p.size(); ++i) {   // the name ends where the parameter list opens
        if (p[i] == '<') ++depth;
        else if (p[i] == '>') --depth;
        else if (p[i] == '(' && depth == 0) {
            p.resize(i);
            break;
        }
    }
    return "(" + p + ")";
}
template <auto K>
const char* kernel_label() {
    static const std::string label = kernel_label_from(typeid(KernelTag<K>).name());
    return label.c_str();
}
}  // namespace tfh

// Kernel arguments beyond the first 512 bytes are not resident when a wave starts: every 64-byte line of them that the
// kernel reaches through a chain of dependent scalar loads costs a miss of its own (a chain through sixteen lines adds
// 1.5 us to an otherwise empty launch, measured on this device).  Called first thing in a kernel whose arguments are
// larger than that, this touches all the later lines at once, so the misses overlap and the loads that follow hit.
template <int BYTES>
__device__ __forceinline__ void prefetch_kernel_arguments() {
    if constexpr (BYTES > 512) {
        const __attribute__((address_space(4))) int* ka = (const __attribute__((address_space(4))) int*)__builtin_amdgcn_kernarg_segment_ptr();
        int sink = 0;
#pragma unroll
        for (int line = 8; line < (BYTES + 63) / 64; ++line) sink += ka[line * 16];
        asm volatile("" ::"s"(sink));
    }
}

#define TFH_LAUNCH_TIMED(kernel, grid, block, lds, st, ...)                                                          \
    do {                                                                                                             \
        const char* label_ = tfh::kernel_label<&kernel>();                                                           \
        tfh::note_kernel(label_);                                                                                    \
        const tfh::ProfEvents pe_ = tfh::prof_take(label_);                                                          \
        if (pe_.start)                                                                                               \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, st, (hipEvent_t)pe_.start, (hipEvent_t)pe_.stop, 0, __VA_ARGS__); \
        else                                                                                                         \
            hipLaunchKernelGGL(kernel, grid, block, lds, st, __VA_ARGS__);                                           \
    } while (0)
