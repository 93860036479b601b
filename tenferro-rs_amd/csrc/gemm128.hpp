// gemm128.hpp -- the 128x128 MFMA contraction kernel (see k_gemm.hip for the algorithm overview).
//
// 512 threads = 8 waves as 4x2, wave tile 32x64, two blocks per CU (<= 128 VGPRs, 76 KB LDS each) so that
// the MFMA phase of one block overlaps the load/store phase of the other.  All operand addressing is a
// uniform 64-bit base plus a per-thread 32-bit byte offset that is constant over the k loop; the base
// advances by one stage per iteration on the scalar unit (single-stride k) or a per-stage table entry is
// added (multi-mode k).  Rows past the matrix edge are read from a clamped (valid) address and never
// stored; only the last, partial k stage is masked to zero.
// f64 accumulators must stay in VGPRs: with AGPR accumulators v_mfma_f64_16x16x4_f64 issues every 130
// cycles instead of 64 on gfx950 (measured), so the kernel is bounded to 128 registers and uses no AGPRs.
#pragma once
#include "gemm_common.hpp"

namespace tfh {
namespace gemm {

// Operand bases are uniform pointers into global memory; saying so lets the compiler emit
// global_load with a scalar base + 32-bit vector offset instead of flat loads with 64-bit vector addresses.
typedef const __attribute__((address_space(1))) char* gptr;
__device__ __forceinline__ gptr as_global(const void* p) { return (gptr)(uintptr_t)p; }
// Pins a (logically uniform) pointer into scalar registers.
__device__ __forceinline__ gptr uniform_ptr(gptr p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (gptr)(((uint64_t)hi << 32) | lo);
}
template <class E> struct RawOf { typedef E type; };
template <> struct RawOf<float2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct RawOf<double2> { typedef double type __attribute__((ext_vector_type(2))); };
template <class E>
__device__ __forceinline__ E gload(gptr base, uint32_t off) {
    typedef typename RawOf<E>::type Raw;
    const Raw r = *reinterpret_cast<const __attribute__((address_space(1))) Raw*>(base + off);
    return __builtin_bit_cast(E, r);
}

template <class R, bool CX>
struct Cfg128 {
    static constexpr int BM = 128, BN = 128;
    static constexpr int BKR = sizeof(R) == 8 ? 16 : 32;  // real k per stage
    static constexpr int BKE = CX ? BKR / 2 : BKR;        // elements of k per stage
    static constexpr int PAD = 16 / sizeof(R);
    static constexpr int PITCH = BKR + PAD;
    static constexpr int BNE = CX ? BN / 2 : BN;          // element columns per tile
    static constexpr int WAVES_M = 2, WAVES_N = 2, NT = 64 * WAVES_M * WAVES_N;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 16, TN = WN / 16;
    static constexpr int MIN_WAVES = 2;   // waves per SIMD the register budget is sized for
    static constexpr int NUA = BM * BKE / NT, NUB = BNE * BKE / NT;
    static constexpr size_t LDS_BYTES = (size_t)2 * (BM + BN) * PITCH * sizeof(R);
};

// Per-thread, loop-invariant description of one operand's share of a stage.  Element u of the thread sits
// at LDS index lds0 + u*LDS_STEP and k index kk0 + u*KK_STEP (compile-time steps).
template <class R, bool CX, int ROWS, int NU, bool KFAST, int RM>
struct TileMap {
    typedef Cfg128<R, CX> C_;
    static constexpr int KK_STEP = KFAST ? 0 : C_::NT / ROWS;
    static constexpr int LDS_STEP = KFAST ? (C_::NT / C_::BKE) * C_::PITCH * RM : KK_STEP * (CX ? 2 : 1);
    uint32_t voff[NU];   // byte offset of element u relative to the (advancing) base
    int lds0, kk0;
    __device__ __forceinline__ int kk(int u) const { return kk0 + u * KK_STEP; }
    __device__ __forceinline__ int lds(int u) const { return lds0 + u * LDS_STEP; }
    __device__ __forceinline__ void init(const Off32& frow, const Off32& fk, int64_t row0, int rows_valid) {
        constexpr int BKE = C_::BKE, NT = C_::NT, PITCH = C_::PITCH;
        const int t = threadIdx.x;
        const int r0 = KFAST ? t / BKE : t % ROWS;
        kk0 = KFAST ? t % BKE : t / ROWS;
        lds0 = r0 * RM * PITCH + (CX ? 2 * kk0 : kk0);   // RM real rows per element row (2 for a complex B)
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const int row = KFAST ? r0 + u * (NT / BKE) : r0;
            const int rc = row < rows_valid ? row : rows_valid - 1;
            voff[u] = off32_of(frow, row0 + rc) + (fk.tab ? 0u : (uint32_t)kk(u) * fk.stride);
        }
    }
};

template <class R, bool CX, bool AKF, bool BKF>
__global__ void __launch_bounds__((Cfg128<R, CX>::NT), (Cfg128<R, CX>::MIN_WAVES)) gemm128_kernel(GemmArgs g) {
    typedef Cfg128<R, CX> C_;
    typedef typename ElemT<R, CX>::type E;
    typedef typename Mfma<R>::acc_t acc_t;
    constexpr int BM = C_::BM, BN = C_::BN, BKR = C_::BKR, BKE = C_::BKE, PITCH = C_::PITCH, BNE = C_::BNE;
    constexpr int TM = C_::TM, TN = C_::TN, NUA = C_::NUA, NUB = C_::NUB;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    R* As = reinterpret_cast<R*>(smem_raw);   // [2][BM][PITCH]
    R* Bs = As + 2 * BM * PITCH;              // [2][BN][PITCH]

    int64_t M = g.M, N = g.N, K = g.K;
    gptr Ap = as_global(g.A32);
    gptr Bp = as_global(g.B32);
    void* Cp = g.C;
    Off32 am = g.am32, ak = g.ak32, bk = g.bk32, bn = g.bn32;
    OffFn cm = g.cm, cn = g.cn;
    int tile_m, tile_n;
    int64_t batch = 0;
    int split = 0;
    if (g.problems) {
        const int4 tm = g.tile_map[blockIdx.x];
        const GroupProblem& p = g.problems[tm.x];
        M = p.M; N = p.N; K = p.K;
        Ap = as_global(p.A); Bp = as_global(p.B); Cp = p.C;
        am.stride = (uint32_t)(p.sam * (int64_t)sizeof(E)); ak.stride = (uint32_t)(p.sak * (int64_t)sizeof(E));
        bk.stride = (uint32_t)(p.sbk * (int64_t)sizeof(E)); bn.stride = (uint32_t)(p.sbn * (int64_t)sizeof(E));
        cm.stride = p.scm; cn.stride = p.scn;
        tile_m = tm.y;
        tile_n = tm.z;
    } else {
        tile_n = blockIdx.x % g.tiles_n;
        tile_m = blockIdx.x / g.tiles_n;
        split = blockIdx.z % g.nsplit;
        batch = blockIdx.z / g.nsplit;
        Ap += off_of(g.ab, batch) * (int64_t)sizeof(E);
        Bp += off_of(g.bb, batch) * (int64_t)sizeof(E);
    }
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BNE;
    const int64_t kbeg = (int64_t)split * g.k_per_split;
    const int64_t kend = (g.nsplit > 1 && kbeg + g.k_per_split < K) ? kbeg + g.k_per_split : K;
    const int rowsA = (int)(M - m0 < BM ? M - m0 : BM), rowsB = (int)(N - n0 < BNE ? N - n0 : BNE);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    TileMap<R, CX, BM, NUA, AKF, 1> ma;
    TileMap<R, CX, BNE, NUB, BKF, (CX ? 2 : 1)> mb;
    ma.init(am, ak, m0, rowsA);
#pragma unroll
    for (int u = 0; u < NUA; ++u) ma.voff[u] += g.problems ? 0u : g.bias_a32;
    mb.init(bn, bk, n0, rowsB);
#pragma unroll
    for (int u = 0; u < NUB; ++u) mb.voff[u] += g.problems ? 0u : g.bias_b32;
    // uniform bases; single-stride k advances them by one stage per iteration
    gptr sa = Ap + (ak.tab ? 0 : (int64_t)(int32_t)ak.stride * kbeg);
    gptr sb = Bp + (bk.tab ? 0 : (int64_t)(int32_t)bk.stride * kbeg);
    const int64_t stepA = ak.tab ? 0 : (int64_t)(int32_t)ak.stride * BKE;
    const int64_t stepB = bk.tab ? 0 : (int64_t)(int32_t)bk.stride * BKE;

    const int wm0 = (wave / C_::WAVES_N) * C_::WM, wn0 = (wave % C_::WAVES_N) * C_::WN;
    const int lrow = lane & 15, lgrp = lane >> 4;

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    E va[NUA], vb[NUB];
    const int64_t klen = kend > kbeg ? kend - kbeg : 0;
    const int64_t nstage = (klen + BKE - 1) / BKE;
    const int rem = (int)(klen - (nstage - 1) * BKE);   // k elements in the last stage (1..BKE)
    const bool ktab = ak.tab != nullptr;               // the host builds k tables for both operands or for none

    // ---- stage loaders ---------------------------------------------------------------------------------------
    // single-stride k, full stage: the invariant offsets against the advancing uniform base
    auto load_fast = [&]() {
        sa = uniform_ptr(sa);
        sb = uniform_ptr(sb);
#pragma unroll
        for (int u = 0; u < NUA; ++u) va[u] = gload<E>(sa, ma.voff[u]);
#pragma unroll
        for (int u = 0; u < NUB; ++u) vb[u] = gload<E>(sb, mb.voff[u]);
        sa += stepA;
        sb += stepB;
    };
    // single-stride k, last stage: k clamped into the range (masked to zero when stored)
    auto load_tail = [&]() {
#pragma unroll
        for (int u = 0; u < NUA; ++u) {
            const int d = ma.kk(u) >= rem ? rem - 1 - ma.kk(u) : 0;
            va[u] = gload<E>(sa, ma.voff[u] + (uint32_t)d * ak.stride);
        }
#pragma unroll
        for (int u = 0; u < NUB; ++u) {
            const int d = mb.kk(u) >= rem ? rem - 1 - mb.kk(u) : 0;
            vb[u] = gload<E>(sb, mb.voff[u] + (uint32_t)d * bk.stride);
        }
    };
    // multi-mode k: per-stage offsets from the tables (k clamped to the last valid index)
    auto load_tab = [&](int64_t s) {
        const int64_t k0 = kbeg + s * BKE;
        uint32_t ka[NUA], kb[NUB];
#pragma unroll
        for (int u = 0; u < NUA; ++u) {
            if (AKF && u > 0) { ka[u] = ka[0]; continue; }
            const int64_t ki = k0 + ma.kk(u);
            ka[u] = ak.tab[ki < kend ? ki : kend - 1];
        }
#pragma unroll
        for (int u = 0; u < NUB; ++u) {
            if (BKF && u > 0) { kb[u] = kb[0]; continue; }
            const int64_t ki = k0 + mb.kk(u);
            kb[u] = bk.tab[ki < kend ? ki : kend - 1];
        }
#pragma unroll
        for (int u = 0; u < NUA; ++u) va[u] = gload<E>(sa, ma.voff[u] + ka[u]);
#pragma unroll
        for (int u = 0; u < NUB; ++u) vb[u] = gload<E>(sb, mb.voff[u] + kb[u]);
    };

    auto store_stage = [&](int buf, bool mask_tail) {
        R* as = As + buf * BM * PITCH;
        R* bs = Bs + buf * BN * PITCH;
#pragma unroll
        for (int u = 0; u < NUA; ++u) {
            E x = va[u];
            const bool ok = !mask_tail || ma.kk(u) < rem;
            if constexpr (CX) {
                x.x = ok ? x.x : R(0);
                x.y = ok ? (g.conj_a ? -x.y : x.y) : R(0);
                *reinterpret_cast<E*>(as + ma.lds(u)) = x;
            } else {
                as[ma.lds(u)] = ok ? x : R(0);
            }
        }
#pragma unroll
        for (int u = 0; u < NUB; ++u) {
            E x = vb[u];
            const bool ok = !mask_tail || mb.kk(u) < rem;
            if constexpr (CX) {
                const R xr = ok ? x.x : R(0);
                const R xi = ok ? (g.conj_b ? -x.y : x.y) : R(0);
                E r0, r1;   // B'[2k][2n] = br, B'[2k+1][2n] = -bi ; B'[2k][2n+1] = bi, B'[2k+1][2n+1] = br
                r0.x = xr; r0.y = -xi;
                r1.x = xi; r1.y = xr;
                *reinterpret_cast<E*>(bs + mb.lds(u)) = r0;            // real row 2n
                *reinterpret_cast<E*>(bs + mb.lds(u) + PITCH) = r1;    // real row 2n+1
            } else {
                bs[mb.lds(u)] = ok ? x : R(0);
            }
        }
    };

    constexpr int NS = BKR / 4;   // MFMA k-steps per stage
    auto compute = [&](int buf) {
        // lane l feeds A[row l%16][k = 4*step + l/16] and B[k = 4*step + l/16][col l%16]
        const R* as = As + buf * BM * PITCH + (wm0 + lrow) * PITCH + lgrp;
        const R* bs = Bs + buf * BN * PITCH + (wn0 + lrow) * PITCH + lgrp;
#pragma unroll
        for (int st = 0; st < NS; ++st) {
            R a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = as[i * 16 * PITCH + 4 * st];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = bs[j * 16 * PITCH + 4 * st];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<R>::run(a[i], b[j], acc[i][j]);
        }
    };

    if (nstage > 0) {
        if (ktab) {
            load_tab(0);
            store_stage(0, nstage == 1);
            __syncthreads();
            int64_t s = 0;
            for (; s + 2 < nstage; ++s) {
                load_tab(s + 1);
                __builtin_amdgcn_sched_barrier(0);
                compute((int)(s & 1));
                __builtin_amdgcn_sched_barrier(0);
                store_stage((int)((s + 1) & 1), false);
                __syncthreads();
            }
            if (s + 1 < nstage) {
                load_tab(s + 1);
                compute((int)(s & 1));
                store_stage((int)((s + 1) & 1), true);
                __syncthreads();
                ++s;
            }
            compute((int)(s & 1));
        } else {
            if (nstage == 1) load_tail();
            else load_fast();
            store_stage(0, nstage == 1);
            __syncthreads();
            int64_t s = 0;
            for (; s + 2 < nstage; ++s) {
                load_fast();
                __builtin_amdgcn_sched_barrier(0);
                compute((int)(s & 1));
                __builtin_amdgcn_sched_barrier(0);
                store_stage((int)((s + 1) & 1), false);
                __syncthreads();
            }
            if (s + 1 < nstage) {
                load_tail();
                compute((int)(s & 1));
                store_stage((int)((s + 1) & 1), true);
                __syncthreads();
                ++s;
            }
            compute((int)(s & 1));
        }
    }

    // ---- epilogue: real column wn0 + 16 j + lrow; for complex, column 2n+p is part p of element n ----------
    const int64_t NR = CX ? 2 * N : N;
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

template <class R, bool CX, bool AKF, bool BKF>
inline void launch_gemm128_variant(const GemmArgs& g, dim3 grid, hipStream_t st) {
    static bool once = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm128_kernel<R, CX, AKF, BKF>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)Cfg128<R, CX>::LDS_BYTES);
        return true;
    }();
    (void)once;
    typedef Cfg128<R, CX> C_;
    const size_t lds = C_::LDS_BYTES;
    const dim3 block(C_::NT);
    hipLaunchKernelGGL((gemm128_kernel<R, CX, AKF, BKF>), grid, block, lds, st, g);
}

template <class R, bool CX>
inline void launch_gemm128_any(const GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    if (akf) {
        if (bkf) launch_gemm128_variant<R, CX, true, true>(g, grid, st);
        else launch_gemm128_variant<R, CX, true, false>(g, grid, st);
    } else {
        if (bkf) launch_gemm128_variant<R, CX, false, true>(g, grid, st);
        else launch_gemm128_variant<R, CX, false, false>(g, grid, st);
    }
}

}  // namespace gemm

// One translation unit per dtype instantiates its four layout variants.
void launch_gemm128_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_f64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_c64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);

}  // namespace tfh
