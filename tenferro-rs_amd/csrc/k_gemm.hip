// k_gemm.hip -- binary tensor contraction on the gfx950 matrix cores: PrimDescriptor::Contract and
// BatchedGemm (tenferro-prims/src/lib.rs:227-239, 156-168) and the grouped (variable-size) form.
//
// C[b, m, n] = alpha * sum_k A[b, m, k] * B[b, k, n] + beta * C, where b, m, n, k are *fused mode
// groups*: each operand element is addressed as base + off_batch(b) + off_row(m) + off_k(k), and every
// off_* is either a single stride or a table built on the device from the group's extents and strides.
// The permutation a contraction implies is therefore applied while the tiles are loaded ("permute on
// load"); nothing is materialised.
//
// Block = 256 threads = 4 waves (2x2), tile BM x BN x BK, double-buffered in LDS with the k index
// contiguous for both operands.  The inner product runs on v_mfma_f64_16x16x4_f64 /
// v_mfma_f32_16x16x4_f32: lane l feeds A[l%16][l/16] and B[l/16][l%16]; a lane reads FOUR consecutive
// k values at once (one or two ds_read_b128) and uses them in four successive MFMAs, which permutes k
// identically for A and B and is harmless under the sum.
// complex128/complex64 run on the real MFMA: the A tile keeps (re, im) interleaved along k, the B tile
// is expanded on its way into LDS to the real 2x2 block [[br, bi], [-bi, br]], so that the real product
// A'(M x 2K) * B'(2K x 2N) is the interleaved complex C(M x N).  conj is a sign flip in the same place.
// MFMA-bound: algorithmic flops = 2*M*N*K (x4 for complex).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <array>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

#include "gemm128.hpp"
#include "gemm_skinny.hpp"
#include "internal.hpp"

namespace tfh {
namespace {

using namespace gemm;

template <class R, bool CX, int BM, int BN>
struct Cfg {
    static constexpr int BKR = sizeof(R) == 8 ? 16 : 32;  // real k per stage
    static constexpr int BKE = CX ? BKR / 2 : BKR;        // elements of k per stage
    static constexpr int PAD = 16 / sizeof(R);
    static constexpr int PITCH = BKR + PAD;
    static constexpr int BNE = CX ? BN / 2 : BN;          // element columns per tile
    // 128x128: 8 waves as 4x2, wave tile 32x64.  64x64: 4 waves as 2x2, wave tile 32x32.
    static constexpr int WAVES_M = BM / 32, WAVES_N = 2;
    static constexpr int NT = 64 * WAVES_M * WAVES_N;     // threads per block
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int TM = WM / 16, TN = WN / 16;
    static constexpr int NUA = BM * BKE / NT, NUB = BNE * BKE / NT;   // elements per thread per stage
    static constexpr size_t TILE_BYTES = (size_t)2 * (BM + BN) * PITCH * sizeof(R);
    static constexpr size_t LDS_BYTES = TILE_BYTES + (size_t)(BM + BNE) * sizeof(int64_t);
    static_assert(BM * BKE % NT == 0 && BNE * BKE % NT == 0, "tile must divide over the block");
    static_assert(NT % BKE == 0 && NT % BM == 0 && NT % BNE == 0, "thread mapping");
};

// Loads this thread's share of one operand tile (ROWS x BKE elements) into registers.  Every address is
// valid (row and k indices are clamped); `kmask` bit u tells whether element u lies inside the k range,
// rows outside the matrix are zeroed when the tile is written to LDS.
template <class E, int ROWS, int BKE, int NU, int NT>
__device__ __forceinline__ void load_tile(E (&v)[NU], uint32_t& kmask, const E* __restrict__ base, const int64_t* rowoff_lds,
                                          int64_t rowoff_fixed, bool kfast, const OffFn& fk, int64_t k0, int64_t kend) {
    const int t = threadIdx.x;
    if (kfast) {
        const int kk = t % BKE;
        const bool kok = k0 + kk < kend;
        const int64_t ko = off_of(fk, kok ? k0 + kk : k0);
        kmask = kok ? 0xffffffffu : 0u;
#pragma unroll
        for (int u = 0; u < NU; ++u) v[u] = base[rowoff_lds[t / BKE + u * (NT / BKE)] + ko];
    } else {
        kmask = 0;
        int64_t ko[NU];
        if (fk.tab) {
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int64_t kidx = k0 + t / ROWS + u * (NT / ROWS);
                const bool kok = kidx < kend;
                kmask |= (kok ? 1u : 0u) << u;
                ko[u] = fk.tab[kok ? kidx : k0];
            }
        } else {
#pragma unroll
            for (int u = 0; u < NU; ++u) {
                const int64_t kidx = k0 + t / ROWS + u * (NT / ROWS);
                const bool kok = kidx < kend;
                kmask |= (kok ? 1u : 0u) << u;
                ko[u] = (kok ? kidx : k0) * fk.stride;
            }
        }
#pragma unroll
        for (int u = 0; u < NU; ++u) v[u] = base[rowoff_fixed + ko[u]];
    }
}

template <class R, bool CX, int BM, int BN>
__global__ void __launch_bounds__((Cfg<R, CX, BM, BN>::NT), 2) gemm_kernel(GemmArgs g) {
    typedef Cfg<R, CX, BM, BN> C_;
    typedef typename ElemT<R, CX>::type E;
    typedef typename Mfma<R>::acc_t acc_t;
    constexpr int BKR = C_::BKR, BKE = C_::BKE, PITCH = C_::PITCH, BNE = C_::BNE, TM = C_::TM, TN = C_::TN;
    constexpr int NUA = C_::NUA, NUB = C_::NUB, NT = C_::NT;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    R* As = reinterpret_cast<R*>(smem_raw);                 // [2][BM][PITCH]
    R* Bs = As + 2 * BM * PITCH;                            // [2][BN][PITCH]
    int64_t* rowA = reinterpret_cast<int64_t*>(smem_raw + C_::TILE_BYTES);   // [BM]  row offsets of this tile
    int64_t* rowB = rowA + BM;                                               // [BNE]

    // ---- which tile ---------------------------------------------------------------------------------
    int64_t M = g.M, N = g.N, K = g.K;
    const void* Ap = g.A;
    const void* Bp = g.B;
    void* Cp = g.C;
    OffFn am = g.am, ak = g.ak, bk = g.bk, bn = g.bn, cm = g.cm, cn = g.cn;
    int tile_m, tile_n;
    int64_t batch = 0;
    int split = 0;
    if (g.problems) {
        const int4 tm = g.tile_map[blockIdx.x];
        const GroupProblem& p = g.problems[tm.x];
        M = p.M; N = p.N; K = p.K;
        Ap = p.A; Bp = p.B; Cp = p.C;
        am.stride = p.sam; ak.stride = p.sak; bk.stride = p.sbk; bn.stride = p.sbn; cm.stride = p.scm; cn.stride = p.scn;
        tile_m = tm.y;
        tile_n = tm.z;
    } else {
        // one-dimensional grid: tiles of one (batch, split) pair are adjacent logical positions
        const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n;
        const uint64_t lb = logical_block(blockIdx.x, gridDim.x);
        const uint32_t lz = (uint32_t)(lb / tiles);
        tile_of((uint32_t)(lb % tiles), g.tiles_m, g.tiles_n, tile_m, tile_n);
        split = (int)(lz % (uint32_t)g.nsplit);
        batch = lz / (uint32_t)g.nsplit;
    }
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BNE;
    const int64_t kbeg = (int64_t)split * g.k_per_split;
    const int64_t kend = (g.nsplit > 1 && kbeg + g.k_per_split < K) ? kbeg + g.k_per_split : K;
    const int rowsA = (int)(M - m0 < BM ? M - m0 : BM), rowsB = (int)(N - n0 < BNE ? N - n0 : BNE);
    const bool a_kfast = g.a_kfast, b_kfast = g.b_kfast;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // row offsets of the tile (clamped to the last valid row so that every load address is valid)
    for (int r = tid; r < BM; r += NT) rowA[r] = off_of(am, m0 + (r < rowsA ? r : rowsA - 1));
    for (int r = tid; r < BNE; r += NT) rowB[r] = off_of(bn, n0 + (r < rowsB ? r : rowsB - 1));
    __syncthreads();
    const E* baseA = reinterpret_cast<const E*>(Ap) + (g.problems ? 0 : off_of(g.ab, batch));
    const E* baseB = reinterpret_cast<const E*>(Bp) + (g.problems ? 0 : off_of(g.bb, batch));
    const int64_t fixedA = rowA[tid % BM], fixedB = rowB[tid % BNE];

    const int wm0 = (wave / C_::WAVES_N) * C_::WM, wn0 = (wave % C_::WAVES_N) * C_::WN;
    const int lrow = lane & 15, lgrp = lane >> 4;

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    E va[NUA], vb[NUB];
    uint32_t maskA = 0, maskB = 0;

    auto store_tiles = [&](int buf) {
        R* as = As + buf * BM * PITCH;
        R* bs = Bs + buf * BN * PITCH;
#pragma unroll
        for (int u = 0; u < NUA; ++u) {
            const int row = a_kfast ? tid / BKE + u * (NT / BKE) : tid % BM;
            const int kk = a_kfast ? tid % BKE : tid / BM + u * (NT / BM);
            const bool ok = row < rowsA && ((maskA >> u) & 1u);
            E x = va[u];
            if constexpr (CX) {
                x.x = ok ? x.x : R(0);
                x.y = ok ? (g.conj_a ? -x.y : x.y) : R(0);
                *reinterpret_cast<E*>(as + row * PITCH + 2 * kk) = x;
            } else {
                as[row * PITCH + kk] = ok ? x : R(0);
            }
        }
#pragma unroll
        for (int u = 0; u < NUB; ++u) {
            const int row = b_kfast ? tid / BKE + u * (NT / BKE) : tid % BNE;
            const int kk = b_kfast ? tid % BKE : tid / BNE + u * (NT / BNE);
            const bool ok = row < rowsB && ((maskB >> u) & 1u);
            E x = vb[u];
            if constexpr (CX) {
                const R xr = ok ? x.x : R(0);
                const R xi = ok ? (g.conj_b ? -x.y : x.y) : R(0);
                E r0, r1;           // B'[2k][2n] = br, B'[2k+1][2n] = -bi ; B'[2k][2n+1] = bi, B'[2k+1][2n+1] = br
                r0.x = xr; r0.y = -xi;
                r1.x = xi; r1.y = xr;
                *reinterpret_cast<E*>(bs + (2 * row) * PITCH + 2 * kk) = r0;
                *reinterpret_cast<E*>(bs + (2 * row + 1) * PITCH + 2 * kk) = r1;
            } else {
                bs[row * PITCH + kk] = ok ? x : R(0);
            }
        }
    };

    const int64_t nstage = kend > kbeg ? (kend - kbeg + BKE - 1) / BKE : 0;
    if (nstage > 0) {
        load_tile<E, BM, BKE, NUA, NT>(va, maskA, baseA, rowA, fixedA, a_kfast, ak, kbeg, kend);
        load_tile<E, BNE, BKE, NUB, NT>(vb, maskB, baseB, rowB, fixedB, b_kfast, bk, kbeg, kend);
        store_tiles(0);
    }
    __syncthreads();
    constexpr int NS = BKR / 4;   // MFMA k-steps per stage
    for (int64_t s = 0; s < nstage; ++s) {
        const int buf = (int)(s & 1);
        const bool more = s + 1 < nstage;
        if (more) {
            load_tile<E, BM, BKE, NUA, NT>(va, maskA, baseA, rowA, fixedA, a_kfast, ak, kbeg + (s + 1) * BKE, kend);
            load_tile<E, BNE, BKE, NUB, NT>(vb, maskB, baseB, rowB, fixedB, b_kfast, bk, kbeg + (s + 1) * BKE, kend);
        }
        // lane l feeds A[row l%16][k = 4*step + l/16] and B[k = 4*step + l/16][col l%16]
        const R* as = As + buf * BM * PITCH + (wm0 + lrow) * PITCH + lgrp;
        const R* bs = Bs + buf * BN * PITCH + (wn0 + lrow) * PITCH + lgrp;
        R a[2][TM], b[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) a[0][i] = as[i * 16 * PITCH];
#pragma unroll
        for (int j = 0; j < TN; ++j) b[0][j] = bs[j * 16 * PITCH];
#pragma unroll
        for (int st = 0; st < NS; ++st) {
            if (st + 1 < NS) {
#pragma unroll
                for (int i = 0; i < TM; ++i) a[(st + 1) & 1][i] = as[i * 16 * PITCH + 4 * (st + 1)];
#pragma unroll
                for (int j = 0; j < TN; ++j) b[(st + 1) & 1][j] = bs[j * 16 * PITCH + 4 * (st + 1)];
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<R>::run(a[st & 1][i], b[st & 1][j], acc[i][j]);
        }
        if (more) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue ---------------------------------------------------------------------------------------
    // real column index inside the tile: wn0 + 16 j + lrow ; for complex, column 2n+p is part p of element n
    const int64_t NR = CX ? 2 * N : N;           // real columns of C
    const int64_t n0r = CX ? 2 * n0 : n0;
    if (g.nsplit > 1) {
        R* P = reinterpret_cast<R*>(g.partial) + ((int64_t)split * g.nbatch + batch) * M * NR;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                int64_t row = m0 + wm0 + 16 * i + Mfma<R>::row(lane, r);
                if (row >= M) continue;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    int64_t col = n0r + wn0 + 16 * j + lrow;
                    if (col < NR) P[row * NR + col] = acc[i][j][r];
                }
            }
        return;
    }
    R* Cb = reinterpret_cast<R*>(Cp) + (g.problems ? 0 : off_of(g.cb, batch)) * (CX ? 2 : 1);
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    int64_t coff[TN];
    bool cok[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        int64_t col = n0r + wn0 + 16 * j + lrow;
        cok[j] = col < NR;
        int64_t n = CX ? col >> 1 : col;
        coff[j] = cok[j] ? off_of(cn, n) * (CX ? 2 : 1) + (CX ? (col & 1) : 0) : 0;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            int64_t row = m0 + wm0 + 16 * i + Mfma<R>::row(lane, r);
            const bool rok = row < M;
            const int64_t roff = rok ? off_of(cm, row) * (CX ? 2 : 1) : 0;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                R v = acc[i][j][r];
                const bool ok = rok && cok[j];
                R* dst = Cb + roff + coff[j];
                if constexpr (CX) {
                    // even lanes hold re, odd lanes hold im of the same element: exchange with the neighbour
                    R other = __shfl_xor(v, 1);
                    R old = (g.use_beta && ok) ? *dst : R(0);
                    R old_other = __shfl_xor(old, 1);
                    const bool im = lane & 1;
                    R re_v = im ? other : v, im_v = im ? v : other;
                    R re_o = im ? old_other : old, im_o = im ? old : old_other;
                    R out = im ? (ar * im_v + ai * re_v) : (ar * re_v - ai * im_v);
                    if (g.use_beta) out += im ? (br * im_o + bi * re_o) : (br * re_o - bi * im_o);
                    if (ok) *dst = out;
                } else {
                    if (ok) {
                        R out = ar * v;
                        if (g.use_beta) out += br * *dst;
                        *dst = out;
                    }
                }
            }
        }
}

// Sums split-K partials in split order and applies alpha/beta.  One thread per element.
template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) splitk_finalize_kernel(GemmArgs g) {
    const int64_t total = g.nbatch * g.M * g.N;
    const int64_t idx = (int64_t)blockIdx.x * THREADS + threadIdx.x;
    if (idx >= total) return;
    const int64_t n = idx % g.N, t = idx / g.N, m = t % g.M, b = t / g.M;
    constexpr int NC = CX ? 2 : 1;
    const R* P = reinterpret_cast<const R*>(g.partial);
    const int64_t plane = g.nbatch * g.M * g.N * NC;
    R sr = 0, si = 0;
    for (int s = 0; s < g.nsplit; ++s) {
        const R* p = P + s * plane + ((b * g.M + m) * g.N + n) * NC;
        sr += p[0];
        if (CX) si += p[1];
    }
    R* dst = reinterpret_cast<R*>(g.C) + (off_of(g.cb, b) + off_of(g.cm, m) + off_of(g.cn, n)) * NC;
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    if (CX) {
        R rr = ar * sr - ai * si, ri = ar * si + ai * sr;
        if (g.use_beta) {
            R cr = dst[0], ci = dst[1];
            rr += br * cr - bi * ci;
            ri += br * ci + bi * cr;
        }
        dst[0] = rr;
        dst[1] = ri;
    } else {
        R r = ar * sr;
        if (g.use_beta) r += br * dst[0];
        dst[0] = r;
    }
}

// Many splits over few outputs (one tile with a very long k): sixteen lanes share an output, lane y adds the partials
// of splits y, y + 16, ... in increasing order and lane 0 adds the sixteen sums in order -- a fixed order, so the
// result does not depend on scheduling.
template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) splitk_finalize_deep_kernel(GemmArgs g) {
    constexpr int SL = 16, OUT = THREADS / SL, NC = CX ? 2 : 1;
    __shared__ R part[SL][OUT][NC];
    const int tx = threadIdx.x % OUT, ty = threadIdx.x / OUT;
    const int64_t total = g.nbatch * g.M * g.N;
    const int64_t idx = (int64_t)blockIdx.x * OUT + tx;
    const bool ok = idx < total;
    const int64_t plane = total * NC;
    R sr = 0, si = 0;
    if (ok) {
        const R* p = reinterpret_cast<const R*>(g.partial) + idx * NC;
        for (int s = ty; s < g.nsplit; s += SL) {
            sr += p[s * plane];
            if (CX) si += p[s * plane + 1];
        }
    }
    part[ty][tx][0] = sr;
    if (CX) part[ty][tx][NC - 1] = si;
    __syncthreads();
    if (ty != 0 || !ok) return;
    sr = 0;
    si = 0;
    for (int y = 0; y < SL; ++y) {
        sr += part[y][tx][0];
        if (CX) si += part[y][tx][NC - 1];
    }
    const int64_t n = idx % g.N, t = idx / g.N, m = t % g.M, b = t / g.M;
    R* dst = reinterpret_cast<R*>(g.C) + (off_of(g.cb, b) + off_of(g.cm, m) + off_of(g.cn, n)) * NC;
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    if (CX) {
        R rr = ar * sr - ai * si, ri = ar * si + ai * sr;
        if (g.use_beta) {
            R cr = dst[0], ci = dst[NC - 1];
            rr += br * cr - bi * ci;
            ri += br * ci + bi * cr;
        }
        dst[0] = rr;
        dst[NC - 1] = ri;
    } else {
        R r = ar * sr;
        if (g.use_beta) r += br * dst[0];
        dst[0] = r;
    }
}

// The same fold with 16-byte accesses, for a C that is contiguous along n: one thread per 16 bytes of a row of C.
template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) splitk_finalize_vec_kernel(GemmArgs g) {
    constexpr int VEC = 16 / sizeof(R), NC = CX ? 2 : 1;
    typedef R Vec __attribute__((ext_vector_type(VEC)));
    const int64_t NR = g.N * NC, nv = NR / VEC;
    const int64_t idx = (int64_t)blockIdx.x * THREADS + threadIdx.x;
    if (idx >= g.nbatch * g.M * nv) return;
    const int64_t v = idx % nv, t = idx / nv, m = t % g.M, b = t / g.M;
    const int64_t plane = g.nbatch * g.M * NR;
    const R* p = reinterpret_cast<const R*>(g.partial) + (b * g.M + m) * NR + v * VEC;
    Vec sum = __builtin_nontemporal_load(reinterpret_cast<const Vec*>(p));
    for (int s = 1; s < g.nsplit; ++s) sum += __builtin_nontemporal_load(reinterpret_cast<const Vec*>(p + s * plane));
    Vec* dst = reinterpret_cast<Vec*>(reinterpret_cast<R*>(g.C) + (off_of(g.cb, b) + off_of(g.cm, m)) * NC + v * VEC);
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    Vec out;
    if constexpr (CX) {
        Vec old = sum;
        if (g.use_beta) old = *dst;
#pragma unroll
        for (int e = 0; e < VEC; e += 2) {
            out[e] = ar * sum[e] - ai * sum[e + 1];
            out[e + 1] = ar * sum[e + 1] + ai * sum[e];
            if (g.use_beta) {
                out[e] += br * old[e] - bi * old[e + 1];
                out[e + 1] += br * old[e + 1] + bi * old[e];
            }
        }
    } else {
        out = sum * ar;
        if (g.use_beta) out += *dst * br;
    }
    *dst = out;
}

// Offsets of every fused index of an axis group (last axis fastest): tab[i] = sum_d idx_d * stride_d.  All
// tables of one contraction are built by one launch (blockIdx.y = table).
constexpr int MAX_TABLES = 13, MAX_TABLE_AXES = 96;
struct TableJobs {
    struct Job {
        void* dst;            // int64 element offsets, or uint32 byte offsets modulo 2^32 when elem_bytes != 0
        int64_t n;
        int32_t first_axis, naxes, elem_bytes, pad;
    } job[MAX_TABLES];
    int64_t dims[MAX_TABLE_AXES], strides[MAX_TABLE_AXES];
};
__global__ void __launch_bounds__(THREADS) build_tables_kernel(TableJobs J) {
    const TableJobs::Job& j = J.job[blockIdx.y];
    const int64_t i = (int64_t)blockIdx.x * THREADS + threadIdx.x;
    if (i >= j.n) return;
    int64_t lin = i, off = 0;
    for (int d = j.first_axis + j.naxes - 1; d >= j.first_axis; --d) {
        const int64_t q = lin / J.dims[d];
        off += (lin - q * J.dims[d]) * J.strides[d];
        lin = q;
    }
    if (j.elem_bytes) reinterpret_cast<uint32_t*>(j.dst)[i] = (uint32_t)(off * j.elem_bytes);
    else reinterpret_cast<int64_t*>(j.dst)[i] = off;
}

int64_t prod(const std::vector<Axis>& ax) {
    int64_t p = 1;
    for (auto& a : ax) p *= a.n;
    return p;
}
int64_t min_stride(const std::vector<Axis>& ax, int slot) {
    int64_t m = INT64_MAX;
    for (auto& a : ax)
        if (a.n > 1 && a.s[slot] != 0) m = std::min<int64_t>(m, std::llabs(a.s[slot]));
    return m;
}
void order_by(std::vector<Axis>& ax, int slot) {
    // slowest first, fastest (smallest stride) last; zero strides first
    std::stable_sort(ax.begin(), ax.end(), [slot](const Axis& x, const Axis& y) {
        int64_t a = std::llabs(x.s[slot]), b = std::llabs(y.s[slot]);
        if (a == 0) a = INT64_MAX;
        if (b == 0) b = INT64_MAX;
        return a > b;
    });
}

template <class R, bool CX, int BM, int BN>
void launch_tile(const GemmArgs& g, dim3 grid, hipStream_t st) {
    size_t lds = Cfg<R, CX, BM, BN>::LDS_BYTES;
    static bool once = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<R, CX, BM, BN>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)Cfg<R, CX, BM, BN>::LDS_BYTES);
        return true;
    }();
    (void)once;
    TFH_LAUNCH_TIMED((gemm_kernel<R, CX, BM, BN>), grid, dim3(Cfg<R, CX, BM, BN>::NT), lds, st, g);
}

void launch_generic64(int dtype, const GemmArgs& g, dim3 grid, hipStream_t st) {
    switch (dtype) {
        case TFH_F32: launch_tile<float, false, 64, 64>(g, grid, st); break;
        case TFH_F64: launch_tile<double, false, 64, 64>(g, grid, st); break;
        case TFH_C64: launch_tile<float, true, 64, 64>(g, grid, st); break;
        default: launch_tile<double, true, 64, 64>(g, grid, st); break;
    }
}
}  // namespace
void launch_gemm_wave(int dtype, const gemm::GemmArgs& g, int64_t nwork, hipStream_t st);   // k_gemm_wave.hip
namespace {
void launch_128(int dtype, const GemmArgs& g, dim3 grid, hipStream_t st, int bn = 128, int bm = 128) {
    if (bm == 64) {
        switch (dtype) {
            case TFH_F32: launch_gemm64x64_f32(g, grid, g.a_kfast, g.b_kfast, st); break;
            case TFH_F64: launch_gemm64x64_f64(g, grid, g.a_kfast, g.b_kfast, st); break;
            case TFH_C64: launch_gemm64x64_c64(g, grid, g.a_kfast, g.b_kfast, st); break;
            default: launch_gemm64x64_c128(g, grid, g.a_kfast, g.b_kfast, st); break;
        }
        return;
    }
    if (bn == 64) {
        switch (dtype) {
            case TFH_F32: launch_gemm128x64_f32(g, grid, g.a_kfast, g.b_kfast, st); break;
            case TFH_F64: launch_gemm128x64_f64(g, grid, g.a_kfast, g.b_kfast, st); break;
            case TFH_C64: launch_gemm128x64_c64(g, grid, g.a_kfast, g.b_kfast, st); break;
            default: launch_gemm128x64_c128(g, grid, g.a_kfast, g.b_kfast, st); break;
        }
        return;
    }
    switch (dtype) {
        case TFH_F32: launch_gemm128_f32(g, grid, g.a_kfast, g.b_kfast, st); break;
        case TFH_F64: launch_gemm128_f64(g, grid, g.a_kfast, g.b_kfast, st); break;
        case TFH_C64: launch_gemm128_c64(g, grid, g.a_kfast, g.b_kfast, st); break;
        default: launch_gemm128_c128(g, grid, g.a_kfast, g.b_kfast, st); break;
    }
}

// Lowest and highest element offset reachable through a set of axes (slot = operand).
void reach(const std::vector<Axis>& ax, int slot, int64_t& lo, int64_t& hi) {
    for (auto& a : ax) {
        if (a.n <= 1) continue;
        int64_t e = (a.n - 1) * a.s[slot];
        if (e < 0) lo += e;
        else hi += e;
    }
}

// 16-byte accesses along an operand's contiguous direction (`lanes`, innermost axis last; `other` is the group the
// lanes do not run along): the innermost axis has stride 1 and either an extent divisible by the vector length, or
// the direction is a single axis of at least one vector -- then the kernel handles the vector that straddles the
// end in its last stage; a row-contiguous operand additionally needs the next k column to lie above the current
// one, because full stages over-read into it.  No alignment beyond the element's is required.
bool vec_ok(int dtype, const std::vector<Axis>& lanes, const std::vector<Axis>& other, bool lanes_are_k, int slot) {
    const int64_t V = 16 / (int64_t)dtype_size(dtype);
    if (V <= 1 || lanes.empty()) return false;
    const Axis& inner = lanes.back();
    if (inner.s[slot] != 1) return false;
    if (inner.n % V == 0) return true;
    if (lanes.size() != 1 || inner.n < V) return false;
    if (lanes_are_k) return true;
    return other.empty() || (other.size() == 1 && (other[0].n == 1 || other[0].s[slot] >= V));
}

// Compute units of the current device (looked up once per device).
uint32_t compute_units() {
    static std::mutex mu;
    static std::map<int, uint32_t> cus;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    std::lock_guard<std::mutex> lk(mu);
    auto it = cus.find(dev);
    if (it != cus.end()) return it->second;
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = (uint32_t)n;
    return (uint32_t)n;
}

// An innermost run of n suits the streaming kernel's units of SKINNY_UNIT consecutive n when it is a whole number of them,
// or long enough that a partly filled last unit costs little (500 = 31 units and a quarter).
bool skinny_run_ok(int64_t n) { return n % SKINNY_UNIT == 0 || n >= 3 * SKINNY_UNIT; }

// A tiny operator (both of its extents at most 8) applied to the last leg of a long tensor -- the long operand's rows
// are contiguous runs of k: the tiny-operator kernel (one thread per element of the long free index) then reads and
// writes with a stride of one row between neighbouring lanes, while the streaming kernel of k_gemm_skinny.hip takes
// whole rows.  Measured on 4M rows (us, tiny | streaming): complex128 8x8 566 | 196 with C contiguous along n and
// 1959 | 189 along m, 4x4 130 | 98 and 412 | 98, 2x4 102 | 82 and 128 | 83, 4x2 73 | 90, 3x3 81 | 85, 2x2 47 | 81 and
// 80 | 81; f64 8x8 195 | 95 and 812 | 92, 4x6 106 | 69, 6x6 120 | 78, 4x4 64 | 69 and 167 | 72, 2x4 50 | 61 and 56 | 64;
// complex64 8x8 193 | 115 and 838 | 100, 4x4 63 | 94 and 187 | 82; f32 8x8 103 | 78 and 333 | 68, 4x4 39 | 69 and
// 76 | 61.  ms: the operator's free extent.
bool last_leg_prefers_streaming(int dtype, const ContractAxes& ax, int64_t M, int64_t N, int64_t K) {
    const bool small_is_a = M <= N;
    const int tslot = small_is_a ? 1 : 0;
    const std::vector<Axis>& small = small_is_a ? ax.M : ax.N;
    const int64_t ms = small_is_a ? M : N;
    if (ms > 8 || K > 8 || K < 2) return false;
    if (K * (int64_t)dtype_size(dtype) % 16 != 0) return false;   // rows of whole 16-byte chunks
    std::vector<Axis> k = ax.K;
    order_by(k, tslot);
    int64_t expect = 1;
    for (int d = (int)k.size() - 1; d >= 0; --d) {
        if (k[d].n > 1 && k[d].s[tslot] != expect) return false;
        expect *= k[d].n;
    }
    const bool rows = min_stride(small, 2) == 1;   // C contiguous along the operator's free index
    switch (dtype) {
        case TFH_C128: return rows ? (ms >= 3 || K >= 4) : K >= 4;
        case TFH_F64: return rows ? (ms >= 4 || K >= 6) : K >= 6;
        case TFH_C64: return rows ? (ms >= 4 || K >= 6) : K >= 6;
        default: return rows ? (ms >= 4 || K >= 8) : K >= 8;
    }
}

int bke_of(int dtype) {
    int bkr = is_double(dtype) ? 16 : 32;
    return is_complex(dtype) ? bkr / 2 : bkr;
}

}  // namespace

// k_gemm_bfirst.hip: batched products whose batch index is the contiguous one in all three tensors (column-major
// "bij,bjk->bik").  try_batch_first returns false when the shape is not one that kernel takes; true when it launched
// (status holds the outcome; *routed, when given, the arguments it launched with).
bool try_batch_first(int dtype, const void* a, const void* b, void* c, const ContractAxes& ax, Scalar alpha, Scalar beta,
                     void* stream, bool conj_a, bool conj_b, int32_t& status, gemm::BfArgs* routed);
int32_t launch_batch_first(int dtype, const gemm::BfArgs& g, void* stream);

namespace {
// A routed launch, kept for repeated calls (ContractRecord): the kernel's argument block as the router built it, with
// what changes from call to call noted beside it -- which input each kernel operand is (the router may have exchanged
// them), the byte distance from a view's first element to the rebased operand base of the large-tile kernel, the size
// of the split-K partials (the workspace is asked for again on every call) and which fold kernel follows.
struct GemmRecord : ContractRecord {
    enum Kind { TILES, BATCH_FIRST } kind = TILES;
    GemmArgs g;
    BfArgs bf;
    uint32_t grid = 0;
    int bn = 0, bm = 0;
    bool use128 = false;
    int src_a = 0, src_b = 1;          // input index of the kernel's A and B
    int64_t d_a32 = 0, d_b32 = 0;      // g.A32 - A, g.B32 - B in bytes
    size_t partial_bytes = 0;
    int fold = 0;                      // 0: none, 1: many splits, 2: 16-byte fold, 3: element-wise fold
    uint32_t fold_grid = 0;
    bool has_tables = false;           // g points into the stream's cache of offset tables
    uint64_t epoch = 0;                // table_epoch() when the record was made
    int device = 0;
};
// The record the router fills while launch_contract runs on this thread (null: none wanted, or the route took a turn
// that cannot be replayed: an operand pack, a conjugated copy, tables built into the workspace).
thread_local GemmRecord* t_record = nullptr;

int32_t launch_contract_impl(int dtype, const void* a, const void* b, void* c, ContractAxes ax, Scalar alpha, Scalar beta,
                             void* stream, bool conj_a, bool conj_b);
void launch_fold(int dtype, int fold, uint32_t fold_grid, const GemmArgs& g, hipStream_t st);
}

// conj: bit 0 = use conj(A), bit 1 = use conj(B) (complex dtypes; ignored for real ones).  The tiled and the streaming
// MFMA kernels conjugate an operand while they stage it (a sign flip on the way into LDS or into the registers), so a
// flagged operand costs nothing.  Shapes that go to the kernels without that flip -- a free group of at most eight
// indices: the tiny-operator, product-reduction and elementwise kernels -- get a conjugated copy of the flagged operand
// first (one pass of the copy kernel over it).
int32_t launch_contract(int dtype, const void* a, const void* b, void* c, ContractAxes ax, Scalar alpha, Scalar beta,
                        void* stream, int conj, std::shared_ptr<ContractRecord>* record) {
    bool ca = (conj & 1) != 0 && is_complex(dtype), cb = (conj & 2) != 0 && is_complex(dtype);
    const int64_t M = prod(ax.M), N = prod(ax.N);
    if ((!ca && !cb) || (M > 8 && N > 8)) {
        if (!record) return launch_contract_impl(dtype, a, b, c, ax, alpha, beta, stream, ca, cb);
        // the router fills the record when the route it takes can be replayed; it stays empty (grid 0) otherwise
        auto rec = std::make_shared<GemmRecord>();
        t_record = rec.get();
        const int32_t e = launch_contract_impl(dtype, a, b, c, ax, alpha, beta, stream, ca, cb);
        t_record = nullptr;
        if (!e && rec->grid) {
            rec->label = tfh_last_kernel();
            *record = std::move(rec);
        }
        return e;
    }
    const size_t eb = dtype_size(dtype);
    void* copies[2] = {nullptr, nullptr};
    auto release = [&]() {
        for (void* p : copies) pool_free(stream, p);
    };
    for (int slot = 0; slot < 2; ++slot) {
        if (!(slot == 0 ? ca : cb)) continue;
        // the operand's axes (those it has a stride on), densely re-strided in the order of their present strides
        std::vector<Axis*> mine;
        for (auto* grp : {&ax.batch, &ax.M, &ax.N, &ax.K})
            for (auto& x : *grp)
                if (x.s[slot] != 0 && x.n > 1) mine.push_back(&x);
        std::stable_sort(mine.begin(), mine.end(), [slot](const Axis* x, const Axis* y) { return std::llabs(x->s[slot]) > std::llabs(y->s[slot]); });
        int64_t elems = 1;
        for (auto* x : mine) elems *= x->n;
        if (int32_t e = pool_alloc(stream, (size_t)std::max<int64_t>(elems, 1) * eb, &copies[slot])) {
            release();
            return e;
        }
        std::vector<Axis> cp;
        int64_t stride = 1;
        for (size_t q = mine.size(); q-- > 0;) {
            cp.push_back(Axis{mine[q]->n, {mine[q]->s[slot], stride, 0}, mine[q]->label});
            mine[q]->s[slot] = stride;
            stride *= mine[q]->n;
        }
        Scalar one, zero;
        one.re = 1;
        if (int32_t e = launch_copy(dtype, slot == 0 ? a : b, copies[slot], cp, one, zero, true, stream)) {
            release();
            return e;
        }
        (slot == 0 ? a : b) = copies[slot];
    }
    const int32_t e = launch_contract_impl(dtype, a, b, c, ax, alpha, beta, stream, false, false);
    release();   // stream-ordered: the next user of these blocks is enqueued after the contraction
    return e;
}

namespace {
int32_t launch_contract_impl(int dtype, const void* a, const void* b, void* c, ContractAxes ax, Scalar alpha, Scalar beta,
                             void* stream, bool conj_a, bool conj_b) {
    const int rb = is_double(dtype) ? 8 : 4;
    const size_t eb = dtype_size(dtype);
    if (((uintptr_t)a % eb) || ((uintptr_t)b % eb) || ((uintptr_t)c % rb))
        return set_error(TFH_ERR_STRIDED, "view base is not aligned to the element size");
    hipStream_t st = (hipStream_t)stream;
    int src_a = 0, src_b = 1;   // which of the caller's inputs the kernel's A and B are (they may be exchanged below)
    int64_t nb = prod(ax.batch), M = prod(ax.M), N = prod(ax.N), K = prod(ax.K);
    if (nb == 0 || M == 0 || N == 0) return TFH_OK;
    for (auto* grp : {&ax.batch, &ax.M, &ax.N})
        for (auto& x : *grp)
            if (x.n > 1 && x.s[2] == 0) return set_error(TFH_ERR_STRIDED, "output view has stride 0 on an axis of extent %lld", (long long)x.n);
    if (K == 0) {
        // empty sum: C = beta*C
        std::vector<Axis> out;
        for (auto* grp : {&ax.batch, &ax.M, &ax.N})
            for (auto& x : *grp) out.push_back(Axis{x.n, {x.s[2], x.s[2], 0}, x.label});
        if (beta.is_zero()) return launch_fill(dtype, c, out, Scalar{0, 0}, stream);
        return launch_copy(dtype, c, c, out, beta, Scalar{0, 0}, false, stream);
    }
    // One free group empty (matrix-vector, vector-matrix, dot and batched dot products): there is nothing for a tile
    // of MFMAs to reuse -- a reduction of the elementwise product, bound by HBM (k_dot.hip)
    // a tiny operator applied to a long tensor (a gate on a leg of a state): a stream over the long operand
    // (on the last leg of the long tensor the streaming kernel further down is usually faster: it is looked at first,
    // and the tiny-operator kernel takes the product if that one cannot)
    bool tiny_deferred = false;
    if (M > 1 && N > 1 && !conj_a && !conj_b) {
        tiny_deferred = last_leg_prefers_streaming(dtype, ax, M, N, K);
        int32_t st_tiny = TFH_OK;
        if (!tiny_deferred && try_tiny_operator(dtype, a, b, c, ax, alpha, beta, stream, st_tiny)) return st_tiny;
    }
    if ((M == 1 || N == 1) && !conj_a && !conj_b) {
        std::vector<Axis> kept, red = ax.K;
        for (auto* grp : {&ax.batch, &ax.M, &ax.N})
            for (auto& x : *grp) kept.push_back(x);
        // Nothing is summed either (a tensor scaled along some of its axes, "asx,x->asx"): the elementwise kernel, with the
        // axes an operand lacks as broadcast axes (stride 0), takes any extents without the reduction machinery
        // ([8191,8193] x [8193]: 1213 -> 220 us; [1000,3,1000] complex128: 65 -> 17 us).  When the extents tile, the
        // product-reduction kernel stays for operands of equal size and for 4-byte elements, where it is 10 % faster.
        auto scale = [&]() {
            const int prof = prof_begin(PROF_CONTRACT, stream);
            const int32_t e = launch_emul(dtype, a, b, c, kept, alpha, beta, stream);
            prof_end(prof, stream);
            return e;
        };
        bool broadcast = false;
        for (auto& x : kept) broadcast = broadcast || (x.n > 1 && (x.s[0] == 0 || x.s[1] == 0));
        if (K == 1 && broadcast && eb >= 8) return scale();
        int32_t st_dot = TFH_OK;
        if (try_dot(dtype, a, b, c, kept, red, alpha, beta, stream, st_dot)) return st_dot;
        if (K == 1) return scale();
        // extents that kernel does not tile: the general reduction kernel with a second operand (axis slots A, C, B),
        // the operand with more elements first.  Shapes beyond its axis limits go on to the tiled kernels.
        auto elems = [&](int slot) {
            double n = 1;
            for (auto* grp : {&kept, &red})
                for (auto& x : *grp)
                    if (x.s[slot] != 0) n *= (double)x.n;
            return n;
        };
        const int pa = elems(1) > elems(0) ? 1 : 0, pb = 1 - pa;
        std::vector<Axis> kept2, red2;
        for (auto& x : kept) kept2.push_back(Axis{x.n, {x.s[pa], x.s[2], x.s[pb]}, x.label});
        for (auto& x : red) red2.push_back(Axis{x.n, {x.s[pa], 0, x.s[pb]}, x.label});
        if (launch_reduce_general(dtype, pa == 0 ? a : b, pa == 0 ? b : a, c, kept2, red2, TFH_REDUCE_SUM, alpha, beta, stream) == TFH_OK)
            return TFH_OK;
        clear_error();
    }
    // the batch index contiguous in all three tensors (column-major "bij,bjk->bik"): a kernel of its own, no packing
    if (M > 1 && N > 1 && nb > 1) {
        int32_t st_bf = TFH_OK;
        GemmRecord* rec = t_record;
        if (try_batch_first(dtype, a, b, c, ax, alpha, beta, stream, conj_a, conj_b, st_bf, rec ? &rec->bf : nullptr)) {
            if (rec && !st_bf) {
                rec->kind = GemmRecord::BATCH_FIRST;
                rec->grid = 1;
                rec->epoch = table_epoch();
                (void)hipGetDevice(&rec->device);
            }
            return st_bf;
        }
    }
    // a long operand against a small one that is too large for the register-resident streaming kernel (k_gemm_thin.hip)
    if (nb == 1 && std::min(M, N) <= 64 && std::max(M, N) >= 4096) {
        int32_t st_thin = TFH_OK;
        if (try_thin_stream(dtype, a, b, c, ax, alpha, beta, stream, conj_a, conj_b, st_thin)) return st_thin;
    }
    // lanes of the epilogue run along n: put C's fastest axis in the N group (swap operands if needed)
    if (min_stride(ax.M, 2) < min_stride(ax.N, 2)) {
        std::swap(a, b);
        std::swap(src_a, src_b);
        std::swap(conj_a, conj_b);
        std::swap(ax.M, ax.N);
        std::swap(M, N);
        for (auto* grp : {&ax.batch, &ax.M, &ax.N, &ax.K})
            for (auto& x : *grp) std::swap(x.s[0], x.s[1]);
    }
    // 128x64 tiles take a thin free group (33..95 real columns) as N: if it is M that is thin, exchange the operands
    // (C is then written along its slower axis, which is the small side of the problem)
    {
        const int ec = is_complex(dtype) ? 2 : 1;
        // (a small operator against a long tensor keeps its orientation: the streaming kernel looks at it below)
        const int64_t per_chunk = 16 / ((int64_t)eb / ec);   // components per 16-byte chunk
        bool streamable = M <= SKINNY_MAX_M && K * ec <= SKINNY_MAX_CHUNKS * per_chunk && N >= 4096;
        if (streamable) {
            // (that kernel works on units of SKINNY_UNIT consecutive n: a long side whose innermost runs are too short
            // for them would end on the 64x64 tiles below, at half the rate of the thin tiles)
            std::vector<Axis> long_side = ax.N;
            order_by(long_side, 2);
            fuse_axes(long_side, 3);
            if (long_side.empty() || !skinny_run_ok(long_side.back().n)) streamable = false;
        }
        if (M < 96 && M * ec >= 33 && N * ec >= 96 && !streamable) {
            std::swap(a, b);
            std::swap(src_a, src_b);
            std::swap(conj_a, conj_b);
            std::swap(ax.M, ax.N);
            std::swap(M, N);
            for (auto* grp : {&ax.batch, &ax.M, &ax.N, &ax.K})
                for (auto& x : *grp) std::swap(x.s[0], x.s[1]);
        }
    }
    // loaders run their lanes along k when the operand is contiguous in k, along the row index otherwise
    bool a_kfast = min_stride(ax.K, 0) <= min_stride(ax.M, 0);
    bool b_kfast = min_stride(ax.K, 1) <= min_stride(ax.N, 1);
    // the order of the k modes is free (it is a sum): follow the memory order of the larger k-contiguous operand
    const bool k_by_b = b_kfast && (!a_kfast || N > M);
    order_by(ax.M, a_kfast ? 2 : 0);
    order_by(ax.N, 2);
    order_by(ax.K, k_by_b ? 1 : 0);
    order_by(ax.batch, 2);

    // An operand whose lanes would stride through memory (its contiguous mode is not the one the loader's lanes
    // run along) is first packed into [batch][rows][k], k contiguous, by the tiled copy kernel: two passes over
    // that operand instead of one 64-byte sector per element in every tile that re-reads it.
    void* packed[2] = {nullptr, nullptr};
    auto release_packed = [&]() {
        for (void* p : packed) pool_free(stream, p);
    };
    for (int slot = 0; slot < 2; ++slot) {
        std::vector<Axis>& rows = slot == 0 ? ax.M : ax.N;
        const bool kfast = slot == 0 ? a_kfast : b_kfast;
        const std::vector<Axis>& lanes = kfast ? ax.K : rows;
        if (lanes.empty() || lanes.back().n == 1) continue;
        if (tiny_deferred) continue;   // (the streaming kernel loads 16-byte chunks, the tiny-operator kernel elements: neither wants a copy)
        const Axis& inner = lanes.back();
        const int64_t run = std::llabs(inner.s[slot]) == 1 ? inner.n * (int64_t)eb : (int64_t)eb;
        if (run >= 32) continue;
        int64_t elems = 1;
        for (auto* grp : {&ax.batch, &rows, &ax.K})
            for (auto& x : *grp)
                if (x.s[slot] != 0) elems *= x.n;
        if (elems * (int64_t)eb > ((int64_t)2 << 30) || elems < 4096) continue;
        void* buf = nullptr;
        if (int32_t e = pool_alloc(stream, (size_t)elems * eb, &buf)) {
            release_packed();
            return e;
        }
        packed[slot] = buf;
        std::vector<Axis> cp;
        int64_t stride = 1;
        std::vector<Axis>* order[3] = {&ax.K, &rows, &ax.batch};   // innermost group first
        for (auto* grp : order)
            for (int d = (int)grp->size() - 1; d >= 0; --d) {
                Axis& x = (*grp)[d];
                if (x.s[slot] == 0) continue;
                cp.push_back(Axis{x.n, {x.s[slot], stride, 0}, x.label});
                x.s[slot] = stride;
                stride *= x.n;
            }
        // (a flagged operand is conjugated by this copy, which it needs anyway)
        if (int32_t e = launch_copy(dtype, slot == 0 ? a : b, buf, cp, Scalar{1, 0}, Scalar{0, 0}, slot == 0 ? conj_a : conj_b, stream)) {
            release_packed();
            return e;
        }
        if (slot == 0) { a = buf; a_kfast = true; conj_a = false; }
        else { b = buf; b_kfast = true; conj_b = false; }
    }
    fuse_axes(ax.M, 3);
    fuse_axes(ax.N, 3);
    fuse_axes(ax.K, 3);
    fuse_axes(ax.batch, 3);

    // A small left operand against a long n whose rows of B are contiguous in k: the streaming kernel of
    // k_gemm_skinny.hip (work units of SKINNY_UNIT consecutive n; the n tables then hold one entry per unit).
    const bool cxd = dtype == TFH_C128;
    const int sk_nc = is_complex(dtype) ? 2 : 1;                  // components per element
    const int64_t sk_q = 16 / ((int64_t)eb / sk_nc);               // components per 16-byte chunk: 2 doubles, 4 floats
    auto whole_chunks = [&](int64_t elems) { return elems * sk_nc % sk_q == 0; };
    // The same product seen from the other side -- the long operand is A and C is contiguous along the few columns
    // of B (C[m][n], n = 0..N-1 adjacent): exchange the operands; the kernel then writes C through a transposing
    // LDS tile ("out_rows").
    bool out_rows = false;
    if (nb == 1 && N <= SKINNY_MAX_M && M >= 4096 && K * sk_nc <= SKINNY_MAX_CHUNKS * sk_q && a_kfast &&
        !k_by_b && !ax.K.empty() && ax.N.size() == 1 && ax.N[0].s[2] == 1 && !ax.M.empty() && skinny_run_ok(ax.M.back().n) &&
        (cxd || (whole_chunks(N) && whole_chunks(K) && (uintptr_t)c % 16 == 0 && (uintptr_t)a % 16 == 0))) {
        bool ok = true;
        int64_t expect = 1;
        for (int d = (int)ax.K.size() - 1; d >= 0; --d) {   // a row of A is one contiguous run of k
            if (ax.K[d].n > 1 && ax.K[d].s[0] != expect) ok = false;
            expect *= ax.K[d].n;
        }
        if (!cxd)
            for (auto& x : ax.M) ok = ok && whole_chunks(x.s[2]) && whole_chunks(x.s[0]);
        const Axis& in = ax.M.back();
        ok = ok && std::llabs(in.s[0]) * SKINNY_UNIT * (int64_t)eb < ((int64_t)1 << 31) &&
             std::llabs(in.s[2]) * SKINNY_UNIT * (int64_t)eb < ((int64_t)1 << 31);
        if (ok) {
            std::swap(a, b);
            std::swap(src_a, src_b);
            std::swap(conj_a, conj_b);
            std::swap(ax.M, ax.N);
            std::swap(M, N);
            std::swap(a_kfast, b_kfast);
            for (auto* grp : {&ax.batch, &ax.M, &ax.N, &ax.K})
                for (auto& x : *grp) std::swap(x.s[0], x.s[1]);
            out_rows = true;
        }
    }
    // ... and with the long operand contiguous along its free index instead of k (the operator on a leg that is not the
    // last, the result carrying that leg last): the same exchange; the kernel parks [k][16 n] and writes through the tile.
    bool out_rows_nfast = false;
    if (!out_rows && nb == 1 && N <= SKINNY_MAX_M && M >= 4096 && K <= SKINNY_MAX_CHUNKS && !a_kfast && !ax.K.empty() &&
        ax.N.size() == 1 && ax.N[0].s[2] == 1 && !ax.M.empty() && ax.M.back().s[0] == 1 && skinny_run_ok(ax.M.back().n) &&
        (cxd || (whole_chunks(N) && (uintptr_t)c % 16 == 0 && (uintptr_t)a % 16 == 0 && whole_chunks(ax.M.back().n)))) {
        bool ok = true;
        if (!cxd) {
            for (size_t d = 0; d + 1 < ax.M.size(); ++d) ok = ok && whole_chunks(ax.M[d].s[0]);
            for (auto& x : ax.M) ok = ok && whole_chunks(x.s[2]);
            for (auto& x : ax.K) ok = ok && whole_chunks(x.s[0]);
        }
        int64_t lo = 0, hi = 0;
        reach(ax.K, 0, lo, hi);
        ok = ok && std::max(-lo, hi) * (int64_t)eb < ((int64_t)1 << 30) &&
             std::llabs(ax.M.back().s[2]) * SKINNY_UNIT * (int64_t)eb < ((int64_t)1 << 31);
        if (ok) {
            std::swap(a, b);
            std::swap(src_a, src_b);
            std::swap(conj_a, conj_b);
            std::swap(ax.M, ax.N);
            std::swap(M, N);
            std::swap(a_kfast, b_kfast);
            for (auto* grp : {&ax.batch, &ax.M, &ax.N, &ax.K})
                for (auto& x : *grp) std::swap(x.s[0], x.s[1]);
            out_rows = out_rows_nfast = true;
        }
    }
    const bool k_rows_b = out_rows || k_by_b;   // the k modes are in the memory order of the (possibly exchanged) B
    bool skinny = nb == 1 && M <= SKINNY_MAX_M && K * sk_nc <= SKINNY_MAX_CHUNKS * sk_q && N >= 4096 &&
                  b_kfast && !out_rows_nfast && !ax.K.empty() && k_rows_b && !ax.N.empty() &&
                  skinny_run_ok(ax.N.back().n) && (out_rows || ax.N.back().s[2] == 1);
    if (skinny) {   // a row of B is one contiguous run of k (A's k order is free: it goes through the k table)
        int64_t expect = 1;
        for (int d = (int)ax.K.size() - 1; d >= 0; --d) {
            if (ax.K[d].n > 1 && ax.K[d].s[1] != expect) skinny = false;
            expect *= ax.K[d].n;
        }
    }
    if (skinny && !cxd) {   // 16-byte chunks of several elements: rows of B must start on 16-byte boundaries and hold whole chunks
        skinny = whole_chunks(K) && (uintptr_t)b % 16 == 0;
        for (auto& x : ax.N) skinny = skinny && whole_chunks(x.s[1]);
    }
    // The same operator on a leg that is not the long tensor's last: B is contiguous along n (as is C), its k strides
    // are whatever they are: the kernel parks a unit as [k][16 n].  The 16-byte loads run along n there: runs of n and
    // the strides above them hold whole chunks.
    bool skinny_nfast = false;
    if (!skinny && nb == 1 && !out_rows && M <= SKINNY_MAX_M && K <= SKINNY_MAX_CHUNKS && N >= 4096 && !b_kfast &&
        !ax.K.empty() && !ax.N.empty() && ax.N.back().s[1] == 1 && ax.N.back().s[2] == 1 && skinny_run_ok(ax.N.back().n)) {
        int64_t lo = 0, hi = 0;
        reach(ax.K, 1, lo, hi);
        skinny_nfast = std::max(-lo, hi) * (int64_t)eb < ((int64_t)1 << 30);
        if (!cxd) {
            skinny_nfast = skinny_nfast && (uintptr_t)b % 16 == 0 && whole_chunks(ax.N.back().n);
            for (size_t d = 0; d + 1 < ax.N.size(); ++d) skinny_nfast = skinny_nfast && whole_chunks(ax.N[d].s[1]);
            for (auto& x : ax.K) skinny_nfast = skinny_nfast && whole_chunks(x.s[1]);
        }
        skinny = skinny_nfast;
    }
    if (out_rows_nfast) skinny = skinny_nfast = true;
    int64_t inner_b = 0, inner_c = 0, skinny_upr = 1;
    int skinny_tail = 0;
    if (skinny) {
        int64_t lo = 0, hi = 0;
        reach(ax.M, 2, lo, hi);
        if (std::max(-lo, hi) * sk_nc >= ((int64_t)1 << 31)) skinny = false;
        if (std::llabs(ax.N.back().s[1]) * SKINNY_UNIT * (int64_t)eb >= ((int64_t)1 << 31)) skinny = false;
    }
    if (skinny) {
        Axis& x = ax.N.back();
        inner_b = x.s[1];
        inner_c = x.s[2];
        skinny_tail = (int)(x.n % SKINNY_UNIT);
        x.n = (x.n + SKINNY_UNIT - 1) / SKINNY_UNIT;   // units per innermost run; the last one holds skinny_tail n (0: all)
        skinny_upr = x.n;
        for (int slot = 0; slot < 3; ++slot) x.s[slot] *= SKINNY_UNIT;
    }
    if (!skinny && tiny_deferred) {
        int32_t st_tiny = TFH_OK;
        if (try_tiny_operator(dtype, a, b, c, ax, alpha, beta, stream, st_tiny)) {
            release_packed();
            return st_tiny;
        }
    }
    int64_t Ntab = N;   // entries of the n tables
    if (skinny) {
        Ntab = 1;
        for (auto& x : ax.N) Ntab *= x.n;
    }

    GemmArgs g;
    std::memset(&g, 0, sizeof g);
    g.A = a; g.B = b; g.C = c;
    g.M = M; g.N = N; g.K = K; g.nbatch = nb;
    g.a_kfast = a_kfast; g.b_kfast = b_kfast;
    g.conj_a = conj_a; g.conj_b = conj_b;
    g.alpha_re = alpha.re; g.alpha_im = alpha.im; g.beta_re = beta.re; g.beta_im = beta.im;
    g.use_beta = !beta.is_zero();

    // tile shape, split-K
    const bool cx = is_complex(dtype);
    const int64_t NR = cx ? 2 * N : N;
    // 128x128 tiles, 128x64 for a thin right-hand side (33..95 real columns), else 64x64
    int bm = 64, bn = 64;
    if (M >= 96 && NR >= 96) bm = bn = 128;
    else if (M >= 96 && NR >= 33) bm = 128;
    auto tiles_for = [&](int tm_, int tn_) { return ((M + tm_ - 1) / tm_) * ((NR + tn_ - 1) / tn_) * nb; };
    const int bke = bke_of(dtype);
    const int64_t kstages = (K + bke - 1) / bke;
    // too few large tiles to fill 256 CUs and too little k to split: fall back to 64x64 tiles
    if (bm == 128 && tiles_for(bm, bn) < 192 && kstages < 32 && tiles_for(64, 64) >= 2 * tiles_for(bm, bn)) bm = bn = 64;
    // large tiles that stay at half a block per CU or less even with the deepest split (512^3 f64: 16 tiles x 4): the
    // 64x64 kernel fills the chip better (18 us against 29 us; from 768^3 on the large tiles win)
    if (bm == 128 && bn == 128 && tiles_for(128, 128) * std::max<int64_t>(1, kstages / 8) <= 128 && tiles_for(64, 64) >= 2 * tiles_for(128, 128))
        bm = bn = 64;
    // f64 / complex128 with at most 64 stages of k (too short for a k split to even out the rounds): 512 large tiles
    // are resident at a time, two per CU; a last round of up to 256 runs one block per CU in 0.62 of a full round's
    // time, a fuller one takes a whole round.  64x64 tiles run 1024 at a time at half the rate per flop, so a round of
    // them costs half a large round, and their last round fills in finer steps.  Estimated times in large rounds, the
    // smaller wins (with a margin: the large tiles read less): 768^3 f64 35.6 -> 30.7 us, 1024^3 56.3 -> 50.8,
    // 2560 x 2048 x 512 (320 large tiles) 131 -> 91, 3072^2 x 512 (576) 199 -> 156, 3584^2 x 256 (784) 138 -> 117;
    // complex128 1024 x 1024 x 256 58 -> 42, 3072 x 1536 x 256 200 -> 156; 480, 768 and 1024 large tiles stay (133 / 138,
    // 202 / 204, 259 / 270 us).  With a longer k the split estimate below evens out the large tiles' rounds, and for
    // 4-byte reals, whose MFMAs take half the time, the small tiles lose (1280^3 f32 48 against 63 us).
    if (bm == 128 && bn == 128 && is_double(dtype) && kstages <= 64 && tiles_for(128, 128) <= 1536 && tiles_for(64, 64) >= 2 * tiles_for(128, 128)) {
        const int64_t t128 = tiles_for(128, 128), t64 = tiles_for(64, 64);
        const int64_t r128 = t128 % 512, r64 = t64 % 1024;
        const double time128 = (double)(t128 / 512) + (r128 == 0 ? 0.0 : (r128 <= 256 ? 0.62 : 1.0));
        const double time64 = 0.5 * ((double)(t64 / 1024) + (r64 == 0 ? 0.0 : 0.5 + 0.5 * (double)r64 / 1024.0));
        if (time64 < 0.9 * time128) bm = bn = 64;
    }
    // thin tiles that cannot reach one block per CU even with the deepest split: 64x64 tiles give twice the blocks
    if (bm == 128 && bn == 64 && tiles_for(128, 64) * std::max<int64_t>(1, kstages / 8) < 256 && tiles_for(64, 64) >= 2 * tiles_for(128, 64))
        bm = 64;
    const int64_t tiles = tiles_for(bm, bn);
    int nsplit = 1;
    if (bm == 128 && tiles >= 32 && kstages >= 16) {
        // 128x128 tiles: 512 blocks are resident at a time (two per CU).  Estimated time of a split count s, in us, from
        // what the kernel measures on this device: a block-stage takes 1.95 us of a CU's matrix cores, a block costs
        // about eight more stages of prologue and epilogue, two blocks sharing a CU overlap fully, one alone leaves
        // latency exposed (x1.7 when the whole launch is one block per CU, x1.25 for the tail of a longer launch), and
        // the fold moves the partials twice.  Picks the s with the least estimate: it
        // trades the idle tail of a partly filled last round against per-block overhead and partial traffic.
        auto estimate = [&](int s_) {
            const double per_block = ((double)((kstages + s_ - 1) / s_) + 8.0) * 1.95 * (double)bn / 128.0;
            const int64_t blocks = tiles * s_, full = blocks / 512, rem = blocks % 512;
            double t = (double)full * 2.0 * per_block;
            if (rem > 256) t += 2.0 * per_block;
            else if (rem > 0) t += (full == 0 ? 1.7 : 1.25) * per_block;
            if (s_ > 1) t += 3.0 + (double)s_ * (double)(nb * M * NR * rb) * 2.0 / 10e6;
            return t;
        };
        const int smax = (int)std::min<int64_t>(16, kstages / 8);
        double best = estimate(1);
        for (int s_ = 2; s_ <= smax; ++s_) {
            const double t = estimate(s_);
            if (t < best * 0.97) {   // a split has to pay for itself clearly
                best = t;
                nsplit = s_;
            }
        }
    } else if (tiles < 256 && kstages >= 8) {
        // Few small tiles: a block of the 64x64 kernel that is alone on its CU takes about 3 us plus 1.25 us per stage,
        // whatever the type (two blocks that share a CU 1.3 times that each); splitting k shortens the blocks, and costs
        // a second launch that reads one partial result per split.  Estimated time in us of a split count, from what
        // those kernels measure on this device (512^3 f64: 21.5 us with 4 splits, 22.9 with 8; 256^3: 17.0 with 2,
        // 13.0 with 4; 64 x 64 x 4096: 25 with 32, 13.3 with 64; 200 x 200 x 2000: 23 with 15, 25 with 31); the count
        // with the least estimate is taken.
        const double out_mb = (double)(nb * M * NR * rb) / 1e6;
        auto estimate = [&](int64_t s_) {
            const double stages = (double)((kstages + s_ - 1) / s_);
            const int64_t blocks = tiles * s_;
            double t = 1.5 + (3.0 + 1.25 * stages) * (blocks > 256 ? 1.3 : 1.0) * (double)((blocks + 511) / 512);
            if (s_ > 1) t += 3.0 + 0.45 * (double)s_ * out_mb;
            return t;
        };
        const int64_t smax = std::min<int64_t>(std::min<int64_t>((512 + tiles - 1) / tiles, kstages / 2), 512);
        double best = estimate(1);
        for (int64_t s_ = 2; s_ <= smax; ++s_) {
            const double t = estimate(s_);
            if (t < best * 0.97) {
                best = t;
                nsplit = (int)s_;
            }
        }
    }
    if (skinny) nsplit = 1;
    // many tiny products (both free extents at most 32): one wave per 32x32 tile, no LDS staging (k_gemm_wave.hip)
    const bool wavek = !skinny && M <= 32 && N <= 32 && nb >= 64 && kstages <= 64;
    if (wavek) nsplit = 1;
    int64_t kps = ((kstages + nsplit - 1) / nsplit) * bke;
    nsplit = (int)((K + kps - 1) / kps);
    g.nsplit = nsplit;
    g.k_per_split = kps;
    g.tiles_m = (int)((M + bm - 1) / bm);
    g.tiles_n = (int)((NR + bn - 1) / bn);
    if (wavek) {
        g.tiles_m = (int)((M + 31) / 32);
        g.tiles_n = (int)((NR + 31) / 32);
    }
    if ((double)g.tiles_m * (double)g.tiles_n * (double)nb * (double)nsplit > 2147483647.0) {
        release_packed();
        return set_error(TFH_ERR_INVALID_ARGUMENT, "contraction too large for one launch (tiles %lld, batch*split %lld)",
                         (long long)g.tiles_m * g.tiles_n, (long long)(nb * nsplit));
    }

    // The 128x128 kernel addresses each operand as a uniform 64-bit base + unsigned 32-bit byte offsets.  A group
    // with a single stride is folded into the base (the tile's first row, the stage's first k), so its offsets only
    // cover one tile or stage -- taken as 128 indices with 8 of slack either way, because a vector that is moved back
    // at a matrix edge can start a few rows before its tile; a multi-axis group goes through a 32-bit table over its
    // whole extent.  Usable when the offsets of
    // an operand span less than 4 GiB: always for operands below 4 GiB, and for larger ones whose long groups have
    // a single stride (anything else takes the generic kernel with 64-bit offsets).
    bool use128 = !skinny && !wavek;   // the large-tile kernel family: 128x128, 128x64 and 64x64 tiles
    int64_t lo_a = 0, hi_a = 0, lo_b = 0, hi_b = 0;
    auto tile_reach = [&](const std::vector<Axis>& grp, int slot, int64_t& lo, int64_t& hi) {
        if (grp.size() == 1) {
            const int64_t s_ = grp[0].s[slot], top = std::min<int64_t>(grp[0].n, 128) + 8;
            if (std::llabs(s_) * (int64_t)eb >= ((int64_t)1 << 31)) use128 = false;   // the kernel steps the base by a signed 32-bit stride
            lo += std::min(-8 * s_, top * s_);
            hi += std::max(-8 * s_, top * s_);
        } else {
            reach(grp, slot, lo, hi);
        }
    };
    tile_reach(ax.M, 0, lo_a, hi_a); tile_reach(ax.K, 0, lo_a, hi_a);
    tile_reach(ax.N, 1, lo_b, hi_b); tile_reach(ax.K, 1, lo_b, hi_b);
    if ((hi_a - lo_a + 1) * (int64_t)eb >= ((int64_t)1 << 32) || (hi_b - lo_b + 1) * (int64_t)eb >= ((int64_t)1 << 32)) use128 = false;
    if (!use128 && bm == 128) {
        bm = bn = 64;
        g.tiles_m = (int)((M + bm - 1) / bm);
        g.tiles_n = (int)((NR + bn - 1) / bn);
    }
    const bool ktab32 = use128 && (ax.K.size() > 1);   // k tables for both operands or for none
    g.vec = use128 && vec_ok(dtype, a_kfast ? ax.K : ax.M, a_kfast ? ax.M : ax.K, a_kfast, 0) &&
            vec_ok(dtype, b_kfast ? ax.K : ax.N, b_kfast ? ax.N : ax.K, b_kfast, 1);

    // workspace: offset tables for every multi-axis group, then the split-K partials.  The 128 kernel reads the
    // operands through 32-bit byte tables (rows of A and B when multi-axis, k of both when k is multi-axis) and
    // only C and the batch offsets through 64-bit element tables.
    struct Want { std::vector<Axis>* grp; int slot; OffFn* fn; int64_t n; bool operand; };
    Want wants[9] = {{&ax.M, 0, &g.am, M, true}, {&ax.K, 0, &g.ak, K, true}, {&ax.K, 1, &g.bk, K, true}, {&ax.N, 1, &g.bn, Ntab, true},
                     {&ax.M, 2, &g.cm, M, false}, {&ax.N, 2, &g.cn, Ntab, false}, {&ax.batch, 0, &g.ab, nb, false},
                     {&ax.batch, 1, &g.bb, nb, false}, {&ax.batch, 2, &g.cb, nb, false}};
    struct Want32 { std::vector<Axis>* grp; int slot; Off32* fn; int64_t n; bool force; };
    Want32 wants32[4] = {{&ax.M, 0, &g.am32, M, false}, {&ax.K, 0, &g.ak32, K, ktab32}, {&ax.K, 1, &g.bk32, K, ktab32}, {&ax.N, 1, &g.bn32, Ntab, false}};
    auto need64 = [&](const Want& w) { return w.grp->size() > 1 && !(use128 && w.operand); };
    auto need32 = [&](const Want32& w) { return use128 && (w.grp->size() > 1 || w.force); };
    size_t table_bytes = 0;
    for (auto& w : wants)
        if (need64(w)) table_bytes += ((size_t)w.n * sizeof(int64_t) + 255) & ~(size_t)255;
    for (auto& w : wants32)
        if (need32(w)) table_bytes += ((size_t)w.n * sizeof(uint32_t) + 255) & ~(size_t)255;
    size_t partial_bytes = nsplit > 1 ? (size_t)nsplit * nb * M * NR * rb : 0;
    // The jobs first, with offsets in place of addresses: their dims and strides are the key under which the finished
    // tables are kept for later calls on this stream.
    size_t cursor = 0;
    TableJobs jobs;
    std::memset(&jobs, 0, sizeof jobs);
    int njobs = 0, naxes = 0;
    int64_t longest = 0;
    std::string key;
    auto add_job = [&](const std::vector<Axis>& grp, int slot, int64_t n, int elem_bytes, size_t entry) {
        TableJobs::Job& j = jobs.job[njobs++];
        const size_t at = cursor;
        j.n = n;
        j.first_axis = naxes;
        j.naxes = (int32_t)grp.size();
        j.elem_bytes = elem_bytes;
        j.pad = 0;
        const int64_t head[3] = {n, (int64_t)grp.size(), elem_bytes};
        key.append((const char*)head, sizeof head);
        for (auto& x : grp) {
            jobs.dims[naxes] = x.n;
            jobs.strides[naxes++] = x.s[slot];
            const int64_t ds[2] = {x.n, x.s[slot]};
            key.append((const char*)ds, sizeof ds);
        }
        longest = std::max(longest, n);
        cursor += ((size_t)n * entry + 255) & ~(size_t)255;
        return at;
    };
    size_t at64[9], at32[4];
    for (int i = 0; i < 9; ++i)
        if (need64(wants[i])) at64[i] = add_job(*wants[i].grp, wants[i].slot, wants[i].n, 0, sizeof(int64_t));
    for (int i = 0; i < 4; ++i)
        if (need32(wants32[i])) at32[i] = add_job(*wants32[i].grp, wants32[i].slot, wants32[i].n, (int)eb, sizeof(uint32_t));
    void* cached = nullptr;
    bool fresh = false;
    if (njobs)
        if (int32_t e = table_cache_get(stream, key, table_bytes, &cached, &fresh)) {
            release_packed();
            return e;
        }
    char* ws = nullptr;
    const size_t ws_bytes = (cached ? 0 : table_bytes) + partial_bytes;
    if (ws_bytes) {
        void* p = nullptr;
        if (int32_t e = workspace(stream, ws_bytes, &p)) {
            release_packed();
            return e;
        }
        ws = (char*)p;
    }
    char* tables = cached ? (char*)cached : ws;
    int jn = 0;
    for (int i = 0; i < 9; ++i) {
        Want& w = wants[i];
        if (need64(w)) {
            jobs.job[jn++].dst = tables + at64[i];
            w.fn->tab = (const int64_t*)(tables + at64[i]);
            w.fn->stride = 0;
        } else {
            w.fn->tab = nullptr;
            w.fn->stride = w.grp->size() == 1 ? (*w.grp)[0].s[w.slot] : 0;
        }
    }
    for (int i = 0; i < 4; ++i) {
        Want32& w = wants32[i];
        if (need32(w)) {
            jobs.job[jn++].dst = tables + at32[i];
            w.fn->tab = (const uint32_t*)(tables + at32[i]);
            w.fn->stride = 0;
        } else {
            w.fn->tab = nullptr;
            w.fn->stride = w.grp->size() == 1 ? (uint32_t)((*w.grp)[0].s[w.slot] * (int64_t)eb) : 0u;
        }
    }
    if (njobs && (!cached || fresh)) {
        hipLaunchKernelGGL(build_tables_kernel, dim3((uint32_t)((longest + THREADS - 1) / THREADS), (uint32_t)njobs), dim3(THREADS), 0, st, jobs);
        if (fresh) table_cache_commit(stream, key);
    }
    if (use128) {
        g.A32 = (const char*)a + lo_a * (int64_t)eb;
        g.B32 = (const char*)b + lo_b * (int64_t)eb;
        g.bias_a32 = (uint32_t)(-lo_a * (int64_t)eb);
        g.bias_b32 = (uint32_t)(-lo_b * (int64_t)eb);
    }
    if (nsplit > 1) g.partial = ws + (cached ? 0 : table_bytes);
    dim3 grid((uint32_t)((int64_t)g.tiles_m * g.tiles_n * nb * nsplit), 1, 1);
    g.one_round = bm == 128 && grid.x <= 2u * compute_units();   // two blocks of the 128-tile kernel fit a CU
    // what a repeated call needs to enqueue this launch again: kept when the route used neither an operand pack nor
    // tables of its own in the workspace (the cached tables stay where they are until they are released)
    GemmRecord* rec = t_record;
    if (rec && (skinny || wavek || packed[0] || packed[1] || (njobs && !cached))) rec = nullptr;
    if (rec) {
        rec->kind = GemmRecord::TILES;
        rec->g = g;
        rec->grid = grid.x;
        rec->bn = bn;
        rec->bm = bm;
        rec->use128 = use128;
        rec->src_a = src_a;
        rec->src_b = src_b;
        rec->d_a32 = use128 ? lo_a * (int64_t)eb : 0;
        rec->d_b32 = use128 ? lo_b * (int64_t)eb : 0;
        rec->partial_bytes = partial_bytes;
        rec->has_tables = njobs != 0;
        rec->epoch = table_epoch();
        (void)hipGetDevice(&rec->device);
    }
    const int prof = prof_begin(PROF_CONTRACT, stream);
    if (skinny) {
        SkinnyArgs sk;
        std::memset(&sk, 0, sizeof sk);
        sk.A = a; sk.B = b; sk.C = c;
        sk.M = (int32_t)M; sk.K = (int32_t)K;
        sk.kc = (int32_t)(K * sk_nc / sk_q);
        sk.use_beta = g.use_beta;
        sk.conj_a = conj_a; sk.conj_b = conj_b;
        sk.out_rows = out_rows;
        sk.plain = alpha.re == 1.0 && alpha.im == 0.0 && beta.is_zero();
        sk.units = Ntab;
        sk.upr = (int32_t)skinny_upr; sk.tail = skinny_tail;
        sk.am = g.am; sk.ak = g.ak; sk.cm = g.cm; sk.bu = g.bn; sk.cu = g.cn;
        sk.bk = g.bk; sk.nfast = skinny_nfast;
        sk.b_in = (int32_t)inner_b; sk.c_in = (int32_t)inner_c;
        sk.alpha_re = alpha.re; sk.alpha_im = alpha.im; sk.beta_re = beta.re; sk.beta_im = beta.im;
        launch_gemm_skinny(dtype, sk, st);
    } else if (wavek) launch_gemm_wave(dtype, g, nb * g.tiles_m * g.tiles_n, st);
    else if (use128) launch_128(dtype, g, grid, st, bn, bm);
    else launch_generic64(dtype, g, grid, st);
    prof_end(prof, stream);
    release_packed();   // stream-ordered: the next user of these blocks is enqueued after this kernel
    if (int32_t e = hip_check(hipGetLastError(), "contraction kernel launch")) return e;
    // the fold of the split-K partials (fixed order: deterministic)
    int fold = 0;
    uint32_t fold_grid = 0;
    if (nsplit > 32) {
        fold = 1;
        fold_grid = (uint32_t)((nb * M * N + 15) / 16);
    } else if (nsplit > 1) {
        // 16-byte fold: C contiguous along n, whole vectors per row, every row of C on a 16-byte boundary
        const int64_t vec = 16 / rb, ncx = cx ? 2 : 1;
        bool fold_vec = !g.cn.tab && g.cn.stride == 1 && NR % vec == 0 && (uintptr_t)c % 16 == 0;
        for (auto* grp : {&ax.M, &ax.batch})
            for (auto& x : *grp) fold_vec = fold_vec && (x.n == 1 || (x.s[2] * ncx) % vec == 0);
        fold = fold_vec ? 2 : 3;
        fold_grid = fold_vec ? (uint32_t)((nb * M * (NR / vec) + THREADS - 1) / THREADS) : (uint32_t)((nb * M * N + THREADS - 1) / THREADS);
    }
    if (rec) {
        rec->fold = fold;
        rec->fold_grid = fold_grid;
    }
    if (fold) {
        launch_fold(dtype, fold, fold_grid, g, st);
        if (int32_t e = hip_check(hipGetLastError(), "split-K finalize launch")) return e;
    }
    return TFH_OK;
}

void launch_fold(int dtype, int fold, uint32_t fold_grid, const GemmArgs& g, hipStream_t st) {
    const dim3 g2(fold_grid), blk(THREADS);
    if (fold == 1) {
        switch (dtype) {
            case TFH_F32: hipLaunchKernelGGL((splitk_finalize_deep_kernel<float, false>), g2, blk, 0, st, g); break;
            case TFH_F64: hipLaunchKernelGGL((splitk_finalize_deep_kernel<double, false>), g2, blk, 0, st, g); break;
            case TFH_C64: hipLaunchKernelGGL((splitk_finalize_deep_kernel<float, true>), g2, blk, 0, st, g); break;
            default: hipLaunchKernelGGL((splitk_finalize_deep_kernel<double, true>), g2, blk, 0, st, g); break;
        }
    } else if (fold == 2) {
        switch (dtype) {
            case TFH_F32: hipLaunchKernelGGL((splitk_finalize_vec_kernel<float, false>), g2, blk, 0, st, g); break;
            case TFH_F64: hipLaunchKernelGGL((splitk_finalize_vec_kernel<double, false>), g2, blk, 0, st, g); break;
            case TFH_C64: hipLaunchKernelGGL((splitk_finalize_vec_kernel<float, true>), g2, blk, 0, st, g); break;
            default: hipLaunchKernelGGL((splitk_finalize_vec_kernel<double, true>), g2, blk, 0, st, g); break;
        }
    } else {
        switch (dtype) {
            case TFH_F32: hipLaunchKernelGGL((splitk_finalize_kernel<float, false>), g2, blk, 0, st, g); break;
            case TFH_F64: hipLaunchKernelGGL((splitk_finalize_kernel<double, false>), g2, blk, 0, st, g); break;
            case TFH_C64: hipLaunchKernelGGL((splitk_finalize_kernel<float, true>), g2, blk, 0, st, g); break;
            default: hipLaunchKernelGGL((splitk_finalize_kernel<double, true>), g2, blk, 0, st, g); break;
        }
    }
}
}  // namespace

// A repeated call: the recorded argument block with this call's addresses and scalars, enqueued as the router
// enqueued it.  Nothing is classified, fused, chosen or allocated on the host (the split-K partials come out of the
// stream's workspace, which has the size from the first call).
bool replay_contract(const ContractRecord& base, int dtype, const void* a, const void* b, void* c, Scalar alpha, Scalar beta,
                     void* stream, int32_t& status) {
    const GemmRecord& r = static_cast<const GemmRecord&>(base);
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev != r.device) return false;
    if (r.kind == GemmRecord::BATCH_FIRST) {
        BfArgs g = r.bf;
        g.A = a; g.B = b; g.C = c;
        g.alpha_re = alpha.re; g.alpha_im = alpha.im; g.beta_re = beta.re; g.beta_im = beta.im;
        status = launch_batch_first(dtype, g, stream);
        return true;
    }
    if (r.has_tables) {
        // the tables the arguments name live in the stream's cache: gone after a release, and a graph that is being
        // captured must pin them, which the router does
        if (r.epoch != table_epoch() || stream_is_capturing(stream)) return false;
    }
    GemmArgs g = r.g;
    const void* in[2] = {a, b};
    g.A = in[r.src_a];
    g.B = in[r.src_b];
    g.C = c;
    if (r.use128) {
        g.A32 = (const char*)g.A + r.d_a32;
        g.B32 = (const char*)g.B + r.d_b32;
    }
    g.alpha_re = alpha.re; g.alpha_im = alpha.im; g.beta_re = beta.re; g.beta_im = beta.im;
    if (r.partial_bytes) {
        void* p = nullptr;
        if ((status = workspace(stream, r.partial_bytes, &p)) != TFH_OK) return true;
        g.partial = p;
    }
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_CONTRACT, stream);
    if (r.use128) launch_128(dtype, g, dim3(r.grid), st, r.bn, r.bm);
    else launch_generic64(dtype, g, dim3(r.grid), st);
    prof_end(prof, stream);
    if ((status = hip_check(hipGetLastError(), "contraction kernel launch")) != TFH_OK) return true;
    if (r.fold) {
        launch_fold(dtype, r.fold, r.fold_grid, g, st);
        status = hip_check(hipGetLastError(), "split-K finalize launch");
    }
    return true;
}

// ---- grouped launch ------------------------------------------------------------------------------------------
struct GroupedState {
    std::vector<int4> tile_map_host;   // (problem, tile_m, tile_n, shape); shape: see gemm128_grouped_kernel; problem -1 = padding
    std::vector<int4> tile_map_uniform;   // every tile 128 x 128 (the scalar-access fallback of the 128 kernel)
    int bm = 128;
    bool shaped = false;               // tile_map_host carries per-tile shapes (128-tile plans)
    std::mutex mu;
    // Problem records (pointers, extents, strides) that earlier calls wrote to the device: a call whose records equal
    // one of these sets launches its contraction on that copy instead of writing its own.  A set is never rewritten
    // (other streams may be reading it); `ready` orders a reader on another stream behind the kernels that wrote it.
    struct Records { std::vector<GroupProblem> host; GroupProblem* dev = nullptr; hipEvent_t ready = nullptr; };
    struct DeviceMaps { int4* shaped = nullptr; int4* uniform = nullptr; std::vector<Records> records; };
    std::map<int, DeviceMaps> maps;    // per device: the tile maps never change after the plan is made, so they are uploaded once
};
constexpr size_t MAX_RECORD_SETS = 8;

void grouped_state_destroy(GroupedState* s) {
    if (!s) return;
    for (auto& kv : s->maps) {
        if (kv.second.shaped) (void)hipFree(kv.second.shaped);
        if (kv.second.uniform) (void)hipFree(kv.second.uniform);
        for (auto& r : kv.second.records) {
            if (r.dev) (void)hipFree(r.dev);
            if (r.ready) (void)hipEventDestroy(r.ready);
        }
    }
    delete s;
}

int32_t grouped_plan_init(tfh_plan& plan) {
    auto* gs = new (std::nothrow) GroupedState();
    if (!gs) return set_error(TFH_ERR_DEVICE, "out of host memory");
    const bool cx = is_complex(plan.dtype);
    const int ec = cx ? 2 : 1;
    struct T { int p, tm, tn, kind; int64_t k; };
    std::vector<T> tiles;
    int64_t small = 0;
    std::vector<std::array<int64_t, 3>> mnk((size_t)plan.n_groups);
    for (int gi = 0; gi < plan.n_groups; ++gi) {
        // extents of the fused groups from the labels: batch modes are not allowed in a grouped plan
        const auto& sa = plan.shapes[(size_t)gi * 3 + 0];
        const auto& sb = plan.shapes[(size_t)gi * 3 + 1];
        int64_t M = 1, N = 1, K = 1;
        for (size_t d = 0; d < plan.modes_a.size(); ++d) {
            uint32_t l = plan.modes_a[d];
            bool in_b = std::find(plan.modes_b.begin(), plan.modes_b.end(), l) != plan.modes_b.end();
            bool in_c = std::find(plan.modes_c.begin(), plan.modes_c.end(), l) != plan.modes_c.end();
            if (in_b && in_c) {
                delete gs;
                return set_error(TFH_ERR_INVALID_ARGUMENT, "grouped contraction does not take batch modes (mode %u)", l);
            }
            if (in_c) M *= sa[d];
            else K *= sa[d];
        }
        for (size_t d = 0; d < plan.modes_b.size(); ++d) {
            uint32_t l = plan.modes_b[d];
            bool in_a = std::find(plan.modes_a.begin(), plan.modes_a.end(), l) != plan.modes_a.end();
            bool in_c = std::find(plan.modes_c.begin(), plan.modes_c.end(), l) != plan.modes_c.end();
            if (in_c) N *= sb[d];
            else if (!in_a) K *= sb[d];
        }
        mnk[(size_t)gi] = {M, N, K};
        if (M < 96 || (cx ? 2 * N : N) < 96) ++small;
    }
    gs->bm = small * 2 > plan.n_groups ? 64 : 128;
    // every problem tiny (M, N <= 32): 32x32 tiles, one wave each (k_gemm_wave.hip)
    bool all_tiny = plan.n_groups >= 64;
    for (int gi = 0; gi < plan.n_groups; ++gi) all_tiny = all_tiny && mnk[(size_t)gi][0] <= 32 && mnk[(size_t)gi][1] <= 32 && mnk[(size_t)gi][2] <= 1024;
    if (all_tiny) gs->bm = 32;
    if (gs->bm != 128) {
        for (int gi = 0; gi < plan.n_groups; ++gi) {
            int64_t M = mnk[(size_t)gi][0], N = mnk[(size_t)gi][1], K = mnk[(size_t)gi][2];
            int64_t NR = cx ? 2 * N : N;
            for (int64_t tm = 0; tm * gs->bm < M; ++tm)
                for (int64_t tn = 0; tn * gs->bm < NR; ++tn) tiles.push_back({gi, (int)tm, (int)tn, 0, K});
        }
        // heaviest tiles (largest K) first, so that the tail of the launch is short
        std::stable_sort(tiles.begin(), tiles.end(), [](const T& x, const T& y) { return x.k > y.k; });
        for (auto& t : tiles) gs->tile_map_host.push_back(make_int4(t.p, t.tm, t.tn, 0));
        plan.grouped = gs;
        return TFH_OK;
    }
    // 128-row tiles.  A last strip of at most 64 rows or 64 real columns gets tiles of that shape instead of a padded
    // 128 x 128 one (extents that are odd multiples of 64 -- half of all extents drawn from {64, 128, ...} -- would
    // otherwise compute 10 % more than the products need): shape 1 = 128 x 64, shape 2 = 64 x 128 (run transposed).
    // Two row panels of a problem (256 rows of A, every full column tile, walked column by column) form a unit: its tiles
    // read the same rows of A and, side by side, the same columns of B; the shorter-running tiles of a last strip are units
    // of their own.  A unit lives on one XCD -- block i of a launch runs on XCD i % 8, each with an L2 of its own.  Measured
    // on the benchmark's 128 blocks: dealing the tiles out one by one in the order of their k, each problem spread over all
    // eight L2s, fetches 2.82 GB for 0.68 GB of operands; units of one row panel 2.09 GB, of two 1.59 GB, of four 1.30 GB,
    // at the same speed within 1 %.  How the units are ordered and dealt out is described where it is done, below.
    struct Unit { std::vector<T> tiles; double cost; double tile_cost; };   // cost of the unit, of one of its tiles
    std::vector<Unit> units;
    // a 128 x 64 tile does half the multiply-adds of a full tile in about 0.63 of its time (measured on thin products)
    const double thin_cost = 0.63;
    for (int gi = 0; gi < plan.n_groups; ++gi) {
        const int64_t M = mnk[(size_t)gi][0], N = mnk[(size_t)gi][1], K = mnk[(size_t)gi][2];
        const int64_t NR = N * ec;
        if (M == 0 || N == 0) continue;
        const int64_t full_m = M / 128, rem_m = M % 128, full_n = NR / 128, rem_n = NR % 128;
        // (a transposed strip is 64 real columns of the transposed product, i.e. 64 / ec rows of this one)
        const bool thin_m = rem_m > 0 && rem_m * ec <= 64, thin_n = rem_n > 0 && rem_n <= 64;
        const int64_t rows128 = full_m + ((rem_m > 0 && !thin_m) ? 1 : 0);   // row panels of 128 (the last one padded)
        const int64_t cols128 = full_n + ((rem_n > 0 && !thin_n) ? 1 : 0);
        const double kcost = (double)((K + 15) / 16 + 8);   // stages plus about eight stages' worth of prologue and epilogue
        const int64_t upanels = 2;   // row panels per unit
        for (int64_t tm0 = 0; tm0 < rows128; tm0 += upanels) {
            Unit u;
            u.cost = 0;
            const int64_t tm1 = std::min(rows128, tm0 + upanels);
            // column by column, so that the unit's row panels read a column of B at the same time
            for (int64_t tn = 0; tn < cols128; ++tn)
                for (int64_t tm = tm0; tm < tm1; ++tm) {
                    u.tiles.push_back({gi, (int)tm, (int)tn, 0, K});
                    u.cost += kcost;
                }
            if (!u.tiles.empty()) {
                u.tile_cost = kcost;
                units.push_back(std::move(u));
            }
            if (thin_n) {   // column strip, a unit of its own (its tiles are shorter): tile_n counts 64-column tiles
                Unit v;
                v.cost = 0;
                v.tile_cost = thin_cost * kcost;
                for (int64_t tm = tm0; tm < tm1; ++tm) {
                    v.tiles.push_back({gi, (int)tm, (int)(2 * cols128), 1, K});
                    v.cost += thin_cost * kcost;
                }
                units.push_back(std::move(v));
            }
        }
        if (thin_m) {   // row strip, transposed: the body's rows are the columns (128 per tile), its 64-wide tile_n counts rows
            Unit u;
            u.cost = 0;
            const int64_t cols = (N + 127) / 128;
            for (int64_t tn = 0; tn < cols; ++tn) {
                u.tiles.push_back({gi, (int)tn, (int)(2 * rows128 * ec), 2, K});
                u.cost += thin_cost * kcost;
            }
            u.tile_cost = thin_cost * kcost;
            units.push_back(std::move(u));
        }
    }
    // Workgroups are dispatched in launch order, position i to XCD i % 8, and position i does not start before position
    // i - 1 has: an XCD whose list holds longer tiles than the others' at the same depth holds all of them back.  So the
    // units are taken in the order of their tiles' duration (longest first; a lone long tile that started late would also
    // run on after everything else has finished) and each goes to the XCD with the least work so far: the eight lists then
    // hold tiles of the same duration at the same depth and the same total.
    std::stable_sort(units.begin(), units.end(), [](const Unit& x, const Unit& y) {
        return x.tile_cost != y.tile_cost ? x.tile_cost > y.tile_cost : x.cost > y.cost;
    });
    std::array<std::vector<T>, XCDS> per_xcd;
    std::array<double, XCDS> load{};
    for (auto& u : units) {
        int best = 0;
        for (int x = 1; x < XCDS; ++x)
            if (load[(size_t)x] < load[(size_t)best]) best = x;
        load[(size_t)best] += u.cost;
        for (auto& t : u.tiles) per_xcd[(size_t)best].push_back(t);
    }
    size_t longest = 0;
    for (auto& v : per_xcd) longest = std::max(longest, v.size());
    for (size_t i = 0; i < longest; ++i)
        for (int x = 0; x < XCDS; ++x) {
            const auto& v = per_xcd[(size_t)x];
            if (i < v.size()) gs->tile_map_host.push_back(make_int4(v[i].p, v[i].tm, v[i].tn, v[i].kind));
            else gs->tile_map_host.push_back(make_int4(-1, 0, 0, -1));
        }
    while (!gs->tile_map_host.empty() && gs->tile_map_host.back().x < 0) gs->tile_map_host.pop_back();
    gs->shaped = true;
    // uniform 128 x 128 tiles for operands that do not allow 16-byte accesses
    for (int gi = 0; gi < plan.n_groups; ++gi) {
        const int64_t M = mnk[(size_t)gi][0], NR = mnk[(size_t)gi][1] * ec, K = mnk[(size_t)gi][2];
        for (int64_t tm = 0; tm * 128 < M; ++tm)
            for (int64_t tn = 0; tn * 128 < NR; ++tn) tiles.push_back({gi, (int)tm, (int)tn, 0, K});
    }
    std::stable_sort(tiles.begin(), tiles.end(), [](const T& x, const T& y) { return x.k > y.k; });
    for (auto& t : tiles) gs->tile_map_uniform.push_back(make_int4(t.p, t.tm, t.tn, 0));
    plan.grouped = gs;
    return TFH_OK;
}

namespace {
// Writes a batch of problem records into device memory from kernel arguments (no host staging buffer,
// so the call is asynchronous and capturable).
constexpr int PROBS_PER_SET = 32;
struct ProblemSet {
    GroupProblem p[PROBS_PER_SET];
    int32_t first, count;
};
__global__ void set_problems_kernel(GroupProblem* dst, ProblemSet s) {
    int i = threadIdx.x;
    if (i < s.count) dst[s.first + i] = s.p[i];
}
}  // namespace

int32_t launch_grouped(const tfh_plan& plan, Scalar alpha, const tfh_view* inputs, Scalar beta, tfh_view* outputs,
                       void* stream) {
    GroupedState* gs = plan.grouped;
    hipStream_t st = (hipStream_t)stream;
    const int dtype = plan.dtype;
    const size_t eb = dtype_size(dtype);
    std::vector<GroupProblem> probs((size_t)plan.n_groups);
    bool ok128 = true, vec = true;
    const int64_t V = 16 / (int64_t)eb;
    // Matrix products (two modes per tensor, one free mode of each operand, one summed): the roles of the axes are the
    // plan's, so a problem's record is read off its views without building and fusing axis lists per problem (a launch
    // of many small problems was bound by this loop: 1024 problems 151 -> 19 us per call on the host).
    int aM = -1, aK = -1, bK = -1, bN = -1, cM = -1, cN = -1;
    bool matrices = plan.modes_a.size() == 2 && plan.modes_b.size() == 2 && plan.modes_c.size() == 2;
    if (matrices) {
        auto pos = [](const std::vector<uint32_t>& m, uint32_t l) { return m[0] == l ? 0 : (m[1] == l ? 1 : -1); };
        for (int d = 0; d < 2; ++d) {
            const uint32_t l = plan.modes_a[(size_t)d];
            const int ib = pos(plan.modes_b, l), ic = pos(plan.modes_c, l);
            if (ic >= 0 && ib < 0) { aM = d; cM = ic; }
            else if (ic < 0 && ib >= 0) { aK = d; bK = ib; }
            else matrices = false;
        }
        for (int d = 0; d < 2; ++d) {
            const uint32_t l = plan.modes_b[(size_t)d];
            const int ia = pos(plan.modes_a, l), ic = pos(plan.modes_c, l);
            if (ic >= 0 && ia < 0) { bN = d; cN = ic; }
            else if (!(ic < 0 && ia >= 0)) matrices = false;
        }
        matrices = matrices && aM >= 0 && aK >= 0 && bK >= 0 && bN >= 0 && cM >= 0 && cN >= 0 && cM != cN && aM != aK && bK != bN;
    }
    for (int gi = 0; gi < plan.n_groups; ++gi) {
        const tfh_view& va = inputs[(size_t)gi * 2 + 0];
        const tfh_view& vb = inputs[(size_t)gi * 2 + 1];
        const tfh_view& vc = outputs[gi];
        if (int32_t e = check_view_against(plan.shapes[(size_t)gi * 3 + 0], va, "grouped input A")) return e;
        if (int32_t e = check_view_against(plan.shapes[(size_t)gi * 3 + 1], vb, "grouped input B")) return e;
        if (int32_t e = check_view_against(plan.shapes[(size_t)gi * 3 + 2], vc, "grouped output")) return e;
        if (matrices) {
            GroupProblem& p = probs[(size_t)gi];
            p.A = view_ptr(va, dtype);
            p.B = view_ptr(vb, dtype);
            p.C = view_ptr(vc, dtype);
            if (((uintptr_t)p.A % eb) || ((uintptr_t)p.B % eb) || ((uintptr_t)p.C % eb))
                return set_error(TFH_ERR_STRIDED, "view base is not aligned to the element size");
            p.M = va.dims[aM]; p.K = va.dims[aK]; p.N = vb.dims[bN];
            // (an extent of 1 has no stride, as in the axis lists, which drop such axes)
            p.sam = p.M == 1 ? 0 : va.strides[aM];
            p.scm = p.M == 1 ? 0 : vc.strides[cM];
            p.sbn = p.N == 1 ? 0 : vb.strides[bN];
            p.scn = p.N == 1 ? 0 : vc.strides[cN];
            p.sak = p.K == 1 ? 0 : va.strides[aK];
            p.sbk = p.K == 1 ? 0 : vb.strides[bK];
            if ((p.M > 1 && p.scm == 0) || (p.N > 1 && p.scn == 0)) return set_error(TFH_ERR_STRIDED, "output view has stride 0");
            if (p.sam < 0 || p.sak < 0 || p.sbk < 0 || p.sbn < 0) ok128 = false;
            if (((p.M - 1) * p.sam + (p.K - 1) * p.sak + 1) * (int64_t)eb >= ((int64_t)1 << 32)) ok128 = false;
            if (((p.N - 1) * p.sbn + (p.K - 1) * p.sbk + 1) * (int64_t)eb >= ((int64_t)1 << 32)) ok128 = false;
            continue;
        }
        ContractAxes ax;
        if (int32_t e = classify_contract(plan.modes_a, va.dims, va.strides, plan.modes_b, vb.dims, vb.strides, plan.modes_c,
                                          vc.dims, vc.strides, ax))
            return e;
        order_by(ax.M, 2);
        order_by(ax.N, 2);
        order_by(ax.K, 0);
        fuse_axes(ax.M, 3);
        fuse_axes(ax.N, 3);
        fuse_axes(ax.K, 3);
        if (ax.M.size() > 1 || ax.N.size() > 1 || ax.K.size() > 1 || !ax.batch.empty())
            return set_error(TFH_ERR_INVALID_ARGUMENT, "grouped contraction: operands of group %d are not plain strided matrices", gi);
        GroupProblem& p = probs[(size_t)gi];
        p.A = view_ptr(va, dtype);
        p.B = view_ptr(vb, dtype);
        p.C = view_ptr(vc, dtype);
        if (((uintptr_t)p.A % eb) || ((uintptr_t)p.B % eb) || ((uintptr_t)p.C % eb))
            return set_error(TFH_ERR_STRIDED, "view base is not aligned to the element size");
        p.M = prod(ax.M); p.N = prod(ax.N); p.K = prod(ax.K);
        p.sam = ax.M.empty() ? 0 : ax.M[0].s[0];
        p.scm = ax.M.empty() ? 0 : ax.M[0].s[2];
        p.sbn = ax.N.empty() ? 0 : ax.N[0].s[1];
        p.scn = ax.N.empty() ? 0 : ax.N[0].s[2];
        p.sak = ax.K.empty() ? 0 : ax.K[0].s[0];
        p.sbk = ax.K.empty() ? 0 : ax.K[0].s[1];
        if ((p.M > 1 && p.scm == 0) || (p.N > 1 && p.scn == 0)) return set_error(TFH_ERR_STRIDED, "output view has stride 0");
        if (p.sam < 0 || p.sak < 0 || p.sbk < 0 || p.sbn < 0) ok128 = false;
        if (((p.M - 1) * p.sam + (p.K - 1) * p.sak + 1) * (int64_t)eb >= ((int64_t)1 << 32)) ok128 = false;
        if (((p.N - 1) * p.sbn + (p.K - 1) * p.sbk + 1) * (int64_t)eb >= ((int64_t)1 << 32)) ok128 = false;
    }
    if (gs->bm == 128 && !ok128)
        return set_error(TFH_ERR_INVALID_ARGUMENT, "grouped contraction: an operand has a negative stride or spans 4 GiB or more");
    if (gs->tile_map_host.empty()) return TFH_OK;
    GemmArgs g;
    std::memset(&g, 0, sizeof g);
    g.nbatch = 1;
    g.nsplit = 1;
    // one loader layout per launch, from the first problem's strides (row-major operands: A contiguous in k, B in n)
    g.a_kfast = std::llabs(probs[0].sak) <= std::llabs(probs[0].sam) || probs[0].M == 1;
    g.b_kfast = std::llabs(probs[0].sbk) <= std::llabs(probs[0].sbn) || probs[0].N == 1;
    // 16-byte accesses: every problem is contiguous along the direction the mapping names, with an extent there that
    // is divisible by the vector length or at least one vector long (the kernel's last stage handles the straddle; a
    // row-contiguous operand then needs its next k column above the current one)
    auto vec_side = [&](bool kfast, int64_t s_lane, int64_t n_lane, int64_t s_other, int64_t n_other) {
        if (s_lane != 1) return false;
        if (n_lane % V == 0) return true;
        if (n_lane < V) return false;
        return kfast || n_other == 1 || s_other >= V;
    };
    for (auto& p : probs) {
        if (V <= 1) vec = false;
        else if (!(g.a_kfast ? vec_side(true, p.sak, p.K, p.sam, p.M) : vec_side(false, p.sam, p.M, p.sak, p.K))) vec = false;
        else if (!(g.b_kfast ? vec_side(true, p.sbk, p.K, p.sbn, p.N) : vec_side(false, p.sbn, p.N, p.sbk, p.K))) vec = false;
    }
    // Tiles of their own shape for the last strips need 16-byte accesses on both operands (or 16-byte elements); in a
    // transposed strip tile the operands change places, so both must also satisfy the other's rule.
    bool shaped = gs->shaped && gs->bm == 128 && (vec || V == 1);
    if (shaped && V > 1)
        for (auto& p : probs) {
            // transposed: the body's A is B (lanes along n when B is row-contiguous), its B is A
            if (!(g.b_kfast ? vec_side(true, p.sbk, p.K, p.sbn, p.N) : vec_side(false, p.sbn, p.N, p.sbk, p.K))) shaped = false;
            if (!(g.a_kfast ? vec_side(true, p.sak, p.K, p.sam, p.M) : vec_side(false, p.sam, p.M, p.sak, p.K))) shaped = false;
        }
    const std::vector<int4>& map_host = shaped ? gs->tile_map_host : (gs->bm == 128 ? gs->tile_map_uniform : gs->tile_map_host);
    // The tile maps never change: one upload per device, the first time the plan runs there (this allocates and waits,
    // so a grouped plan is run once eagerly before it is captured into a graph, like every other first call).
    int4* map_dev = nullptr;
    {
        std::lock_guard<std::mutex> lk(gs->mu);
        int dev = 0;
        if (int32_t e = hip_check(hipGetDevice(&dev), "hipGetDevice")) return e;
        GroupedState::DeviceMaps& dm = gs->maps[dev];
        int4*& slot = (shaped || gs->bm != 128) ? dm.shaped : dm.uniform;
        if (!slot) {
            const size_t nb = map_host.size() * sizeof(int4);
            // (into a local pointer first: the slot must never name a map that was not filled)
            int4* fresh = nullptr;
            if (int32_t e = hip_check(hipMalloc((void**)&fresh, std::max<size_t>(nb, 16)), "hipMalloc(tile map)")) return e;
            if (int32_t e = hip_check(hipMemcpy(fresh, map_host.data(), nb, hipMemcpyHostToDevice), "upload tile map")) {
                (void)hipFree(fresh);
                return e;
            }
            slot = fresh;
        }
        map_dev = slot;
    }
    // The problem records belong to the call: they go into this stream's workspace (stream order keeps them intact until
    // the contraction that reads them has run), written from kernel arguments -- no host staging, capturable.  Two
    // executes of one plan on two streams therefore never share records.
    // A call that repeats an earlier one (same buffers, same strides: an iteration that reuses its storage) finds its
    // records on the device already and launches nothing but the contraction (config 4: four launches and 12 us less
    // per step).  New records get a copy of their own, up to MAX_RECORD_SETS per plan and device; beyond that, and while
    // the stream is being captured (nothing may be allocated then), they go into the workspace as described above.
    const size_t rec_bytes = sizeof(GroupProblem) * (size_t)plan.n_groups;
    GroupProblem* problems_dev = nullptr;
    auto write_records = [&](GroupProblem* dst) {
        for (int first = 0; first < plan.n_groups; first += PROBS_PER_SET) {
            ProblemSet s;
            s.first = first;
            s.count = std::min(PROBS_PER_SET, plan.n_groups - first);
            std::memcpy(s.p, probs.data() + first, sizeof(GroupProblem) * (size_t)s.count);
            hipLaunchKernelGGL(set_problems_kernel, dim3(1), dim3(64), 0, st, dst, s);
        }
    };
    if (!stream_is_capturing(stream)) {
        // (the lock is held until a new set's writes and its event are enqueued: another thread that finds the set waits
        // for an event that has been recorded)
        std::lock_guard<std::mutex> lk(gs->mu);
        int dev = 0;
        if (int32_t e = hip_check(hipGetDevice(&dev), "hipGetDevice")) return e;
        GroupedState::DeviceMaps& dm = gs->maps[dev];
        for (auto& r : dm.records)
            if (std::memcmp(r.host.data(), probs.data(), rec_bytes) == 0) {
                if (int32_t e = hip_check(hipStreamWaitEvent(st, r.ready, 0), "hipStreamWaitEvent")) return e;
                problems_dev = r.dev;
                break;
            }
        if (!problems_dev && dm.records.size() < MAX_RECORD_SETS) {
            GroupedState::Records r;
            if (hipMalloc((void**)&r.dev, rec_bytes) == hipSuccess && hipEventCreateWithFlags(&r.ready, hipEventDisableTiming) == hipSuccess) {
                r.host = probs;
                write_records(r.dev);
                if (int32_t e = hip_check(hipEventRecord(r.ready, st), "hipEventRecord")) {
                    // the kernels that write the records are enqueued already: they must finish before the block goes
                    (void)hipStreamSynchronize(st);
                    (void)hipFree(r.dev);
                    (void)hipEventDestroy(r.ready);
                    return e;
                }
                problems_dev = r.dev;
                dm.records.push_back(std::move(r));
            } else {
                (void)hipGetLastError();
                if (r.dev) (void)hipFree(r.dev);
            }
        }
    }
    if (!problems_dev) {
        void* ws = nullptr;
        if (int32_t e = workspace(stream, rec_bytes, &ws)) return e;
        problems_dev = (GroupProblem*)ws;
        write_records(problems_dev);
    }
    // 64 x 64 tiles run on the large-tile kernel as well when its 32-bit offsets suffice
    const bool large64 = gs->bm == 64 && ok128;
    g.vec = (gs->bm == 128 || large64) && vec;
    g.alpha_re = alpha.re; g.alpha_im = alpha.im; g.beta_re = beta.re; g.beta_im = beta.im;
    g.use_beta = !beta.is_zero();
    g.problems = problems_dev;
    g.tile_map = map_dev;
    dim3 grid((uint32_t)map_host.size(), 1, 1);
    const int prof = prof_begin(PROF_CONTRACT, stream);
    if (gs->bm == 32) launch_gemm_wave(dtype, g, (int64_t)map_host.size(), st);
    else if (shaped) {
        switch (dtype) {
            case TFH_F32: launch_gemm128_grouped_f32(g, grid, g.a_kfast, g.b_kfast, st); break;
            case TFH_F64: launch_gemm128_grouped_f64(g, grid, g.a_kfast, g.b_kfast, st); break;
            case TFH_C64: launch_gemm128_grouped_c64(g, grid, g.a_kfast, g.b_kfast, st); break;
            default: launch_gemm128_grouped_c128(g, grid, g.a_kfast, g.b_kfast, st); break;
        }
    } else if (gs->bm == 128) launch_128(dtype, g, grid, st);
    else if (large64) launch_128(dtype, g, grid, st, 64, 64);
    else launch_generic64(dtype, g, grid, st);
    prof_end(prof, stream);
    return hip_check(hipGetLastError(), "grouped contraction launch");
}

}  // namespace tfh
