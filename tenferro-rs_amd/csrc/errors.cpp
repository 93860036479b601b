// errors.cpp -- thread-local record of the last failure, mirroring tenferro_device::Error
// (tenferro-device/src/lib.rs:108-159), plus the small formatting helpers of the C ABI.
#include <cstring>

#include "internal.hpp"

namespace tfh {
namespace {
thread_local tfh_error_info g_err = {};

void format_dims(char* buf, size_t cap, const int64_t* d, int n) {
    size_t pos = 0;
    pos += snprintf(buf + pos, cap - pos, "[");
    for (int i = 0; i < n && pos < cap; ++i) pos += snprintf(buf + pos, cap - pos, i ? ", %lld" : "%lld", (long long)d[i]);
    if (pos < cap) snprintf(buf + pos, cap - pos, "]");
}
}  // namespace

void clear_error() { g_err.status = TFH_OK; g_err.message[0] = 0; g_err.n_expected = g_err.n_got = 0; }

int32_t set_error(int32_t status, const char* fmt, ...) {
    clear_error();
    g_err.status = status;
    const char* prefix = status == TFH_ERR_DEVICE ? "device error: "
                         : status == TFH_ERR_INVALID_ARGUMENT ? "invalid argument: "
                         : status == TFH_ERR_STRIDED ? "strided: "
                         : "";
    size_t off = snprintf(g_err.message, sizeof g_err.message, "%s", prefix);
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err.message + off, sizeof g_err.message - off, fmt, ap);
    va_end(ap);
    return status;
}

int32_t set_shape_mismatch(const int64_t* expected, int n_expected, const int64_t* got, int n_got) {
    clear_error();
    g_err.status = TFH_ERR_SHAPE_MISMATCH;
    g_err.n_expected = n_expected > TFH_MAX_RANK ? TFH_MAX_RANK : n_expected;
    g_err.n_got = n_got > TFH_MAX_RANK ? TFH_MAX_RANK : n_got;
    memcpy(g_err.expected, expected, sizeof(int64_t) * g_err.n_expected);
    memcpy(g_err.got, got, sizeof(int64_t) * g_err.n_got);
    char e[200], g[200];
    format_dims(e, sizeof e, expected, g_err.n_expected);
    format_dims(g, sizeof g, got, g_err.n_got);
    // "shape mismatch: expected {expected:?}, got {got:?}" (tenferro-device/src/lib.rs:111)
    snprintf(g_err.message, sizeof g_err.message, "shape mismatch: expected %s, got %s", e, g);
    return TFH_ERR_SHAPE_MISMATCH;
}

int32_t set_rank_mismatch(int64_t expected, int64_t got) {
    clear_error();
    g_err.status = TFH_ERR_RANK_MISMATCH;
    g_err.n_expected = g_err.n_got = 1;
    g_err.expected[0] = expected;
    g_err.got[0] = got;
    // "rank mismatch: expected {expected}, got {got}" (tenferro-device/src/lib.rs:119)
    snprintf(g_err.message, sizeof g_err.message, "rank mismatch: expected %lld, got %lld", (long long)expected, (long long)got);
    return TFH_ERR_RANK_MISMATCH;
}

int32_t set_no_compatible_device(int32_t space_kind, int64_t space_id, int32_t op_kind) {
    static const char* kinds[] = {"Contract", "BatchedGemm", "Reduce", "Trace", "Permute", "ElementwiseMul"};
    clear_error();
    g_err.status = TFH_ERR_NO_COMPATIBLE_DEVICE;
    g_err.n_expected = 2;   // the memory space: (tfh_space_kind, space id)
    g_err.expected[0] = space_kind;
    g_err.expected[1] = space_kind == TFH_SPACE_GPU_MEMORY ? space_id : 0;
    g_err.n_got = 1;        // the operation: tfh_op_kind
    g_err.got[0] = op_kind;
    const char* op = op_kind >= 0 && op_kind <= TFH_KIND_ELEMENTWISE_MUL ? kinds[op_kind] : "?";
    // "no compatible compute device for {op:?} on {space:?}" (tenferro-device/src/lib.rs:134)
    if (space_kind == TFH_SPACE_GPU_MEMORY)
        snprintf(g_err.message, sizeof g_err.message, "no compatible compute device for %s on GpuMemory { space_id: %lld }", op, (long long)space_id);
    else
        snprintf(g_err.message, sizeof g_err.message, "no compatible compute device for %s on MainMemory", op);
    return TFH_ERR_NO_COMPATIBLE_DEVICE;
}
}  // namespace tfh

extern "C" {

void tfh_last_error(tfh_error_info* out) {
    if (out) *out = tfh::g_err;
}

const char* tfh_status_name(int32_t status) {
    switch (status) {
        case TFH_OK: return "Ok";
        case TFH_ERR_SHAPE_MISMATCH: return "ShapeMismatch";
        case TFH_ERR_RANK_MISMATCH: return "RankMismatch";
        case TFH_ERR_DEVICE: return "DeviceError";
        case TFH_ERR_NO_COMPATIBLE_DEVICE: return "NoCompatibleComputeDevice";
        case TFH_ERR_CROSS_MEMORY_SPACE: return "CrossMemorySpaceOperation";
        case TFH_ERR_INVALID_ARGUMENT: return "InvalidArgument";
        case TFH_ERR_STRIDED: return "Strided";
        default: return "Unknown";
    }
}

const char* tfh_version(void) { return "tenferro-hip 0.1 (gfx950)"; }

size_t tfh_dtype_size(int32_t dtype) { return tfh::dtype_size(dtype); }

int32_t tfh_compute_device_format(int32_t kind, int64_t device_id, char* buf, size_t cap) {
    // Display for ComputeDevice (tenferro-device/src/lib.rs:64-72)
    const char* name = kind == TFH_DEVICE_CPU ? "cpu" : kind == TFH_DEVICE_CUDA ? "cuda" : kind == TFH_DEVICE_HIP ? "hip" : nullptr;
    if (!name || !buf || cap == 0) return tfh::set_error(TFH_ERR_INVALID_ARGUMENT, "unknown compute device kind %d", kind);
    snprintf(buf, cap, "%s:%lld", name, (long long)device_id);
    return TFH_OK;
}

}  // extern "C"
