// k_gemm_wave.hip -- batches of tiny products (PrimDescriptor::BatchedGemm / Contract with batch modes,
// tenferro-prims/src/lib.rs:156-168, 227-239, when M and N are at most 32): one WAVE per 32x32 output tile.
//
// A block-level tile (64x64 or 128x128, staged through LDS, two barriers per stage) computes one tile per tiny problem
// and spends its time in per-tile latency (100 000 products of 8x8x8 f64: 0.53 ms for 154 MB of data).  Here a wave owns
// a 32x32 tile (2x2 blocks of v_mfma_*_16x16x4) of one batch entry, loads its operands straight from global memory in
// the MFMA operand layout -- lane l = 16 g + j feeds A[row j][k = k0 + g] and B[k = k0 + g][col j] -- with bounds
// masks instead of padding, and never waits for another wave: thousands of independent problems are in flight.
// Addressing is the general one of the tiled kernels (base + off_batch + off_row + off_k, strides or tables), complex
// runs on the real MFMA with A interleaved along k and B expanded (B'[2k][2n] = br, B'[2k+1][2n] = -bi,
// B'[2k][2n+1] = bi, B'[2k+1][2n+1] = br).  Bound by load latency and L1/L2 bandwidth, not by the matrix cores.
#include <hip/hip_runtime.h>

#include "gemm_common.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

using namespace gemm;

template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) gemm_wave_kernel(GemmArgs g, int64_t nwork) {
    typedef typename ElemT<R, CX>::type E;
    typedef typename Mfma<R>::acc_t acc_t;
    constexpr int EC = CX ? 2 : 1;
    const int lane = threadIdx.x & 63, j = lane & 15, gq = lane >> 4;
    const int64_t work = (int64_t)blockIdx.x * (THREADS / 64) + (threadIdx.x >> 6);
    if (work >= nwork) return;   // whole waves leave; there is no block-level synchronisation below
    int64_t M = g.M, N = g.N, K = g.K;
    OffFn am = g.am, ak = g.ak, bk = g.bk, bn = g.bn, cm = g.cm, cn = g.cn;
    const E* A;
    const E* B;
    R* Cb;
    int tile_m, tile_n;
    if (g.problems) {   // grouped launch: one record per problem, one map entry per tile
        const int4 tm = g.tile_map[work];
        const GroupProblem& p = g.problems[tm.x];
        M = p.M; N = p.N; K = p.K;
        A = reinterpret_cast<const E*>(p.A);
        B = reinterpret_cast<const E*>(p.B);
        Cb = reinterpret_cast<R*>(p.C);
        am = OffFn{nullptr, p.sam}; ak = OffFn{nullptr, p.sak}; bk = OffFn{nullptr, p.sbk};
        bn = OffFn{nullptr, p.sbn}; cm = OffFn{nullptr, p.scm}; cn = OffFn{nullptr, p.scn};
        tile_m = tm.y;
        tile_n = tm.z;
    } else {
        const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
        const int64_t batch = work / tiles;
        const int tile = (int)(work - batch * tiles);
        tile_m = tile % g.tiles_m;
        tile_n = tile / g.tiles_m;
        A = reinterpret_cast<const E*>(g.A) + off_of(g.ab, batch);
        B = reinterpret_cast<const E*>(g.B) + off_of(g.bb, batch);
        Cb = reinterpret_cast<R*>(g.C) + off_of(g.cb, batch) * EC;
    }
    const int64_t NR = N * EC, KR = K * EC;
    const int64_t m0 = (int64_t)tile_m * 32, n0r = (int64_t)tile_n * 32;

    // this lane's two rows of A and two (real) columns of B; -1 marks the ones outside the matrices
    int64_t ra[2], cb[2];
    int pb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t row = m0 + j + 16 * i;
        ra[i] = row < M ? off_of(am, row) : -1;
        const int64_t col = n0r + j + 16 * i;
        pb[i] = CX ? (int)(col & 1) : 0;
        cb[i] = col < NR ? off_of(bn, CX ? col >> 1 : col) : -1;
    }
    acc_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) acc[i][jb] = acc_t{0, 0, 0, 0};
    // a problem of at most 16 rows or 16 real columns leaves the second block of that side empty: its MFMAs are skipped
    // (the same for every lane of the wave; 8x8x8 f64 issues four of the sixteen)
    const bool rows2 = m0 + 16 < M, cols2 = n0r + 16 < NR;

    // four k steps (16 real k) per iteration: their loads are issued together, then the sixteen MFMAs
    for (int64_t k0 = 0; k0 < KR; k0 += 16) {
        R av[4][2], bv[4][2];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (k0 + 4 * u >= KR) break;   // (the same for every lane: a short k ends the iteration early)
            const int64_t kk = k0 + 4 * u + gq;
            const bool kok = kk < KR;
            const int64_t ke = kok ? (CX ? kk >> 1 : kk) : 0;
            const int q = CX ? (int)(kk & 1) : 0;
            const int64_t ka = off_of(ak, ke), kb = off_of(bk, ke);
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                av[u][i] = R(0);
                if (kok && ra[i] >= 0) {
                    const R* p = reinterpret_cast<const R*>(A + ra[i] + ka);
                    R x = p[CX ? q : 0];
                    if (CX && q && g.conj_a) x = -x;
                    av[u][i] = x;
                }
                bv[u][i] = R(0);
                if (kok && cb[i] >= 0) {
                    const R* p = reinterpret_cast<const R*>(B + cb[i] + kb);
                    if constexpr (CX) {
                        const R br = p[0], bi = g.conj_b ? -p[1] : p[1];
                        bv[u][i] = q == 0 ? (pb[i] ? bi : br) : (pb[i] ? br : -bi);
                    } else {
                        bv[u][i] = p[0];
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (k0 + 4 * u >= KR) break;
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int jb = 0; jb < 2; ++jb)
                    if ((i == 0 || rows2) && (jb == 0 || cols2)) acc[i][jb] = Mfma<R>::run(av[u][i], bv[u][jb], acc[i][jb]);
        }
    }

    // ---- epilogue: the same arithmetic as the tiled kernels; real column n0r + 16 jb + j
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    int64_t coff[2];
    bool cok[2];
#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
        const int64_t col = n0r + 16 * jb + j;
        cok[jb] = col < NR;
        coff[jb] = cok[jb] ? off_of(cn, CX ? col >> 1 : col) * EC + (CX ? (col & 1) : 0) : 0;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t row = m0 + 16 * i + Mfma<R>::row(lane, r);
            const bool rok = row < M;
            const int64_t roff = rok ? off_of(cm, row) * EC : 0;
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                R v = acc[i][jb][r];
                const bool ok = rok && cok[jb];
                R* dst = Cb + roff + coff[jb];
                if constexpr (CX) {
                    // even lanes hold re, odd lanes im of one element: exchange with the neighbour
                    const R other = __shfl_xor(v, 1);
                    const R old = (g.use_beta && ok) ? *dst : R(0);
                    const R old_other = __shfl_xor(old, 1);
                    const bool im = lane & 1;
                    const R re_v = im ? other : v, im_v = im ? v : other;
                    const R re_o = im ? old_other : old, im_o = im ? old : old_other;
                    R out = im ? (ar * im_v + ai * re_v) : (ar * re_v - ai * im_v);
                    if (g.use_beta) out += im ? (br * im_o + bi * re_o) : (br * re_o - bi * im_o);
                    if (ok) *dst = out;
                } else if (ok) {
                    R out = ar * v;
                    if (g.use_beta) out += br * *dst;
                    *dst = out;
                }
            }
        }
}

}  // namespace

// g.tiles_m / g.tiles_n count 32x32 tiles (32 real columns); nwork = batches * tiles.
void launch_gemm_wave(int dtype, const gemm::GemmArgs& g, int64_t nwork, hipStream_t st) {
    const dim3 grid((uint32_t)((nwork + THREADS / 64 - 1) / (THREADS / 64))), block(THREADS);
    switch (dtype) {
        case TFH_F32: TFH_LAUNCH_TIMED((gemm_wave_kernel<float, false>), grid, block, 0, st, g, nwork); break;
        case TFH_F64: TFH_LAUNCH_TIMED((gemm_wave_kernel<double, false>), grid, block, 0, st, g, nwork); break;
        case TFH_C64: TFH_LAUNCH_TIMED((gemm_wave_kernel<float, true>), grid, block, 0, st, g, nwork); break;
        default: TFH_LAUNCH_TIMED((gemm_wave_kernel<double, true>), grid, block, 0, st, g, nwork); break;
    }
}

}  // namespace tfh
