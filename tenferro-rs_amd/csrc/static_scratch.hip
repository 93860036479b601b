// static_scratch.hip -- tfh_execute_static: TensorPrims::execute for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
//
// tfh_execute takes the device scratch of a call -- offset tables, split-K partials, partial sums of a split
// reduction, a packed copy of an operand -- from per-stream buffers that it allocates and grows on demand.  Here the
// same kernels get that scratch from one fixed array in device memory that is part of the library's code object, so the
// call allocates and frees nothing.  Each device the library runs on holds its own copy of the array (at its own
// address) until the process ends.
//
// Nothing in the array has to start at zero: the kernels write every table entry and every partial they later read
// (there are no counters or flags in it), so the contents a previous call left behind are simply overwritten.  All calls
// on one device share the array; two calls that overlap in time on one device -- from two threads, or on two streams --
// race on it.
#include <hip/hip_runtime.h>

#include <exception>
#include <mutex>

#include "internal.hpp"

static __device__ __align__(256) unsigned char scratch[TFH_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex g_mu;
void* g_scratch_ptr[MAX_DEVICES];   // device address of `scratch` on each device, looked up once per device

// `scratch` names the host-side stand-in of the array; the memory itself is reached only through the address the
// runtime reports for the device that is current.
int32_t scratch_address(void** out) {
    int dev = 0;
    if (int32_t e = tfh::hip_check(hipGetDevice(&dev), "hipGetDevice")) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return tfh::set_error(TFH_ERR_DEVICE, "device %d is beyond the %d this library tracks", dev, MAX_DEVICES);
    std::lock_guard<std::mutex> lk(g_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (int32_t e = tfh::hip_check(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return e;
        if (!p) return tfh::set_error(TFH_ERR_DEVICE, "hipGetSymbolAddress(scratch) returned a null address");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return TFH_OK;
}
}  // namespace

extern "C" {

size_t tfh_static_scratch_bytes(void) { return TFH_STATIC_SCRATCH_BYTES; }

int32_t tfh_execute_static(const tfh_plan* plan, const void* alpha, const tfh_view* inputs, int32_t n_inputs, const void* beta,
                           tfh_view* output, tfh_stream stream) {
    void* base = nullptr;
    if (int32_t e = scratch_address(&base)) return e;
    // (the arena ends with this scope whatever happens inside: an exception out of the host code below -- an allocation
    // failure of a std::vector, say -- must not leave later calls of this thread carving from the shared array)
    struct ArenaScope {
        ArenaScope(void* b, size_t n) { tfh::arena_begin(b, n); }
        ~ArenaScope() { tfh::arena_end(); }
    } scope(base, TFH_STATIC_SCRATCH_BYTES);
    try {
        return tfh_execute(plan, alpha, inputs, n_inputs, beta, output, stream);
    } catch (const std::exception& ex) {
        return tfh::set_error(TFH_ERR_DEVICE, "tfh_execute_static: %s", ex.what());
    } catch (...) {
        return tfh::set_error(TFH_ERR_DEVICE, "tfh_execute_static: unknown exception");
    }
}

}  // extern "C"
