// gemm_common.hpp -- argument block and MFMA wrappers shared by the contraction kernels.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace tfh {
namespace gemm {

constexpr int THREADS = 256;

typedef double d4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

struct OffFn {
    const int64_t* tab;  // offsets per fused index, or null
    int64_t stride;      // used when tab == null
};
__device__ __forceinline__ int64_t off_of(const OffFn& f, int64_t i) { return f.tab ? f.tab[i] : i * f.stride; }

// Byte offsets modulo 2^32 for the 128x128 kernel: the host rebases each operand to its lowest reachable
// address and guarantees that the reachable span is below 4 GiB, so sums of wrapped components are exact.
struct Off32 {
    const uint32_t* tab;  // byte offsets per fused index, or null
    uint32_t stride;      // byte stride (wrapped) when tab == null
};
__device__ __forceinline__ uint32_t off32_of(const Off32& f, int64_t i) { return f.tab ? f.tab[i] : (uint32_t)i * f.stride; }

struct GroupProblem {   // one problem of a grouped launch (plain strided matrices)
    const void* A;
    const void* B;
    void* C;
    int64_t M, N, K;
    int64_t sam, sak, sbk, sbn, scm, scn;
};

// One launch of the batch-first kernel (k_gemm_bfirst.hip): batched products whose batch index is the contiguous one.
struct BfArgs {
    const void* A;
    const void* B;
    void* C;
    int64_t nb;                              // extent of the contiguous batch axis
    int64_t nbo;                             // extent of an outer batch axis (1: none)
    int64_t M, N, K;
    int64_t sam, sak, sbk, sbn, scm, scn;    // element strides of the row, column and k axes
    int64_t sao, sbo, sco;                   // element strides of the outer batch axis
    int32_t tiles_m, tiles_n, groups;        // groups of NB batch entries
    int32_t conj_a, conj_b, use_beta;
    double alpha_re, alpha_im, beta_re, beta_im;
};

struct GemmArgs {
    const void* A;
    const void* B;
    void* C;
    int64_t M, N, K, nbatch;
    OffFn am, ak, bk, bn, cm, cn, ab, bb, cb;
    int32_t a_kfast, b_kfast, conj_a, conj_b;
    int32_t nsplit, use_beta;
    int64_t k_per_split;
    void* partial;
    int32_t tiles_m, tiles_n;
    double alpha_re, alpha_im, beta_re, beta_im;
    // 128x128 kernel only: operand bases moved to the lowest reachable address + wrapped byte offsets
    const char* A32;
    const char* B32;
    Off32 am32, ak32, bk32, bn32;
    uint32_t bias_a32, bias_b32;   // byte distance from the rebased base back to element 0
    int32_t vec;                   // both operands allow 16-byte accesses along their contiguous direction
    const GroupProblem* problems;  // grouped launch when non-null
    const int4* tile_map;          // per block: (problem, tile_m, tile_n, 0)
    int32_t one_round;             // 128x128 kernel: every block of the launch is resident at once (see the main loop)
};

// Workgroups are handed to the eight XCDs (each with its own L2) round-robin in launch order.  logical_block()
// maps a launch position to a logical position such that every XCD works through one contiguous range of
// logical positions; tile_of() walks the tiles of one matrix eight tile rows at a time (tile row fastest), so
// that the ~64 blocks resident on an XCD form a compact patch that shares its A rows and B columns in that L2.
constexpr int XCDS = 8;
__host__ __device__ __forceinline__ uint64_t logical_block(uint64_t flat, uint64_t total) {
    const uint64_t per = total / XCDS, rem = total % XCDS, xcd = flat % XCDS, pos = flat / XCDS;
    return (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + pos;
}
__device__ __forceinline__ void tile_of(uint32_t x, int tiles_m, int tiles_n, int& tile_m, int& tile_n) {
    constexpr uint32_t GM = 8;
    const uint32_t span = GM * (uint32_t)tiles_n, first = (x / span) * GM, r = x % span;
    const uint32_t gsz = (uint32_t)tiles_m - first < GM ? (uint32_t)tiles_m - first : GM;
    tile_m = (int)(first + r % gsz);
    tile_n = (int)(r / gsz);
}

template <class R> struct Mfma;
template <> struct Mfma<double> {
    typedef d4 acc_t;
    __device__ static __forceinline__ d4 run(double a, double b, d4 c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    // accumulator register r of lane l holds row (l/16) + 4r, column l%16
    __device__ static __forceinline__ int row(int lane, int r) { return (lane >> 4) + 4 * r; }
};
template <> struct Mfma<float> {
    typedef f4 acc_t;
    __device__ static __forceinline__ f4 run(float a, float b, f4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    // accumulator register r of lane l holds row 4*(l/16) + r, column l%16
    __device__ static __forceinline__ int row(int lane, int r) { return 4 * (lane >> 4) + r; }
};

template <class R, bool CX> struct ElemT;
template <> struct ElemT<float, false> { typedef float type; };
template <> struct ElemT<double, false> { typedef double type; };
template <> struct ElemT<float, true> { typedef float2 type; };
template <> struct ElemT<double, true> { typedef double2 type; };



}  // namespace gemm
}  // namespace tfh
