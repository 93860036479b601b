// gemm_skinny.hpp -- argument block of the contraction kernel for a small left operand (k_gemm_skinny.hip).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "gemm_common.hpp"

namespace tfh {
namespace gemm {

constexpr int SKINNY_UNIT = 16;        // consecutive n (rows of B, columns of C) per work unit
constexpr int SKINNY_MAX_M = 32;       // rows of A
constexpr int SKINNY_MAX_CHUNKS = 32;  // 16-byte chunks per row of B: 64 doubles or 128 floats (half as many complex elements)

struct SkinnyArgs {
    const void* A;
    const void* B;
    void* C;
    int32_t M, K;            // rows of A, elements of k
    int32_t kc;              // 16-byte chunks per row of B: K for complex128, K/2 for f64 and complex64, K/4 for f32
    int32_t conj_a, conj_b, use_beta, plain;   // plain: alpha == 1 and beta == 0
    int32_t out_rows;        // C is contiguous along m (the rows of A), not along n: a unit's results are transposed in LDS
    int64_t units;           // work units: (outer extents of n) x upr
    int32_t upr, tail;       // units per innermost run of n; n in the last unit of each run (0: every unit is full)
    OffFn am, ak, cm;        // element offsets of A's rows and k, of C's rows
    OffFn bu, cu;            // element offset of a unit's first n in B and in C
    OffFn bk;                // nfast: element offset of k in B
    int32_t nfast;           // B is contiguous along n instead of k (complex128, C along n)
    int32_t b_in, c_in;      // element stride between consecutive n inside a unit, in B and in C
    double alpha_re, alpha_im, beta_re, beta_im;
};

}  // namespace gemm

void launch_gemm_skinny(int dtype, const gemm::SkinnyArgs& s, hipStream_t st);
}  // namespace tfh
