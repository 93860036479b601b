// gemm128.hpp -- the 128x128 MFMA contraction kernel (see k_gemm.hip for the algorithm overview).
//
// 256 threads = 4 waves as 2x2, wave tile 64x64 (4x4 MFMA blocks), two blocks per CU so that the MFMA
// phase of one block overlaps the load/store phase of the other.  All operand addressing is a uniform
// 64-bit base plus a per-thread 32-bit byte offset that is constant over the k loop; the base advances by
// one stage per iteration on the scalar unit (single-stride k) or a per-stage table entry is added
// (multi-mode k).  Rows past the matrix edge are read from a clamped (valid) address and never stored;
// only the last, partial k stage is masked to zero.
//
// A stage of an operand is ROWS x 128 bytes of k in LDS, rows 128 bytes apart with no padding: eight 16-byte chunks per
// row, chunk c of row r stored at position c ^ (r & 7) ^ ((r >> 3) & 3).  The LDS of gfx950 serves a 16-byte read of a
// wave in four cycles (256 bytes per cycle) only if, in each half of the wave, lanes 0-7 together with lanes 24-31 and
// lanes 8-15 together with lanes 16-23 touch sixteen different 16-byte bank groups of the 64 banks; otherwise it falls
// back to eight lanes per cycle.  A 16-byte write goes eight lanes at a time over 128 bytes of banks.  (Measured with
// single-pattern loops on a saturated LDS: 4.4 against 8.0 cycles per wave read, 13 against 16 per wave write.)  With
// this position function the fragment reads below (sixteen consecutive rows, lane groups two chunks apart) meet the
// read rule and the stores of both loader shapes (eight lanes along k of one row, or eight rows 1, 2 or 4 apart at one
// k) the write rule.  A loader moves V elements per access (V = 16 bytes / element when the operand's
// contiguous direction allows it, else 1):
//   k-contiguous operand  : one global load of V consecutive k of one row, one LDS store;
//   row-contiguous operand: V loads (V consecutive k) of V consecutive rows each, transposed in registers
//                           into V LDS stores of V consecutive k.
// A lane reads its fragments as whole chunks (two 16-byte LDS reads per 16-row block and stage) and feeds
// MFMA number (h, c) with k = (2*(lane/16) + h)*CH + c -- a permutation of k applied to A and B alike.
//
// f64 accumulators must stay in VGPRs: with AGPR accumulators v_mfma_f64_16x16x4_f64 issues every 130
// cycles instead of 64 on gfx950 (measured), so the kernel is sized to 256 VGPRs and uses no AGPRs.
#pragma once
#include "gemm_common.hpp"
#include "launch.hpp"

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
template <class R, int N> struct RawVec { typedef R type __attribute__((ext_vector_type(N))); };
template <class R> struct RawVec<R, 1> { typedef R type; };
template <class R, int N> struct alignas(sizeof(R) * N) Pack { R v[N]; };
// Global loads promise only element alignment (gfx950 executes an under-aligned global_load_dwordx4), so an operand
// whose rows start at odd element offsets still takes the 16-byte path.
template <class R, int N> struct RawVecU { typedef R type __attribute__((ext_vector_type(N), aligned(sizeof(R)))); };
template <class R> struct RawVecU<R, 1> { typedef R type; };
template <class R, int N>
__device__ __forceinline__ Pack<R, N> gload_pack(gptr base, uint32_t off) {
    typedef typename RawVecU<R, N>::type Raw;
    const Raw r = *reinterpret_cast<const __attribute__((address_space(1))) Raw*>(base + off);
    Pack<R, N> out;
    if constexpr (N == 1) out.v[0] = r;
    else {
#pragma unroll
        for (int i = 0; i < N; ++i) out.v[i] = r[i];
    }
    return out;
}
// x or -x by an XOR of the sign bit
__device__ __forceinline__ double flip_sign(double x, bool flip) {
    return __builtin_bit_cast(double, __builtin_bit_cast(uint64_t, x) ^ (flip ? 0x8000000000000000ull : 0ull));
}
__device__ __forceinline__ float flip_sign(float x, bool flip) {
    return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, x) ^ (flip ? 0x80000000u : 0u));
}
template <class R, int N>
__device__ __forceinline__ void lds_store_pack(R* p, const R (&x)[N]) {
    typedef typename RawVec<R, N>::type Raw;
    Pack<R, N> t;
#pragma unroll
    for (int i = 0; i < N; ++i) t.v[i] = x[i];
    *reinterpret_cast<Raw*>(p) = __builtin_bit_cast(Raw, t);
}

// BNV: real columns per tile, 128 or 64 (a thin right-hand side: 33..95 real columns); BMV: rows per tile, 128, or 64 for
// products with too few large tiles to fill the device (64 x 64 tiles: wave tile 32 x 32, four blocks per CU)
template <class R, bool CX, int BNV = 128, int BMV = 128>
struct Cfg128 {
    static constexpr int BM = BMV, BN = BNV;
    static constexpr int BKR = 128 / sizeof(R);           // real k per stage: 128 bytes per row
    static constexpr int EC = CX ? 2 : 1;                 // reals per element
    static constexpr int BKE = BKR / EC;                  // elements of k per stage
    static constexpr int CH = 16 / sizeof(R);             // reals per 16-byte chunk
    static constexpr int VMAX = CH / EC;                  // elements per 16-byte chunk
    static constexpr int PITCH = BKR;                     // rows are not padded: the chunk swizzle alone spreads the banks
    static constexpr int BNE = BN / EC;                   // element columns per tile
    static constexpr int WAVES_M = 2, WAVES_N = 2, NT = 64 * WAVES_M * WAVES_N;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 16, TN = WN / 16;
    static constexpr int MIN_WAVES = BMV == 64 ? 4 : 2;   // waves per SIMD the register budget is sized for
    static constexpr size_t LDS_BYTES = (size_t)2 * (BM + BN) * PITCH * sizeof(R);
    static_assert((TM == 4 && (TN == 4 || TN == 2)) || (TM == 2 && TN == 2), "wave tiles are four or two 16-row blocks high and wide");
    static_assert(BKR / CH == 8, "eight 16-byte chunks per row");
    // position of a row's chunks: see the layout note at the top of the file
    __device__ static __forceinline__ int swizzle(int rr) { return (rr & 7) ^ ((rr >> 3) & 3); }
    // LDS index of real k `rk` in real row `rr`
    __device__ static __forceinline__ int lds_idx(int rr, int rk) { return rr * PITCH + (((rk / CH) ^ swizzle(rr)) * CH) + rk % CH; }
};

// Per-thread, loop-invariant description of one operand's share of a stage (ROWS element rows x BKE k).
//   KFAST : load l covers row rq + l*RP, k elements kq .. kq+V-1
//   else  : load l = p*V + j covers rows rq .. rq+V-1 at k element (p*KP + kq)*V + j
template <class R, bool CX, int ROWS, bool KFAST, int V, int RM, int BNV = 128>
struct OperandMap {
    typedef Cfg128<R, CX, BNV> C_;
    static constexpr int EC = C_::EC, PN = V * EC;
    static constexpr int KV = C_::BKE / V;             // KFAST: loads per row
    static constexpr int RP = C_::NT / KV;             // KFAST: rows per pass
    static constexpr int RVN = ROWS / V;               // row-contiguous: row groups per k
    static constexpr int KP = C_::NT / RVN;            // row-contiguous: k patches per pass
    static constexpr int NP = KFAST ? ROWS / RP : C_::BKE / (KP * V);
    static constexpr int NL = KFAST ? NP : NP * V;     // loads per thread and stage
    static_assert(NP >= 1 && (KFAST ? NP * RP == ROWS : NP * KP * V == C_::BKE), "operand tile must divide over the block");
    typedef Pack<R, PN> P;
    uint32_t voff[NL];   // byte offset of load l relative to the (advancing) base
    int kq, rq;
    int lds0;            // LDS index of this thread's first 16-byte store (unit 0); the other units derive from it
    // Last stage only.  A vector that straddles the end of its contiguous direction (k past `rem` for a k-contiguous
    // operand, rows past the matrix edge for a row-contiguous one) is loaded from a window moved back to end exactly
    // at the boundary -- nothing is read past the operand -- and its elements are moved up by the same amount when
    // they are stored.  Full stages need none of this: there such a vector only over-reads into the operand's next
    // column, which exists.
    int row_shift;
    __device__ __forceinline__ int kk(int l) const { return KFAST ? kq : ((l / V) * KP + kq) * V + (l % V); }
    __device__ __forceinline__ void init(const Off32& frow, const Off32& fk, int64_t row0, int rows_valid) {
        const int t = threadIdx.x;
        if (KFAST) { kq = (t % KV) * V; rq = t / KV; }
        else { rq = (t % RVN) * V; kq = t / RVN; }
        row_shift = (!KFAST && rq < rows_valid && rq + V > rows_valid) ? rq + V - rows_valid : 0;
        lds0 = C_::lds_idx(rq * RM, (KFAST ? kq : kq * V) * EC);
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            const int row = KFAST ? rq + l * RP : rq;
            // a load wholly past the edge is redirected to the last valid one
            const int rc = row < rows_valid ? row : rows_valid - (KFAST ? 1 : V);
            voff[l] = off32_of(frow, row0 + rc) + (fk.tab ? 0u : (uint32_t)kk(l) * fk.stride);
        }
    }
    // single-stride k, full stage
    __device__ __forceinline__ void load_fast(P (&x)[NL], gptr base) const {
#pragma unroll
        for (int l = 0; l < NL; ++l) x[l] = gload_pack<R, PN>(base, voff[l]);
    }
    // single-stride k, last stage with `rem` valid k: k redirected into the range (masked to zero when stored)
    // The 32-bit offsets are unsigned distances from `base`.  With fewer than V valid k the window of a k-contiguous
    // operand starts before this stage (inside the previous one): the base itself is moved back by that much, so
    // that no offset goes below zero.
    __device__ __forceinline__ void load_tail(P (&x)[NL], gptr base, int rem, uint32_t kstride, uint32_t rowstride) const {
        const uint32_t back = (uint32_t)(-row_shift) * rowstride;
        const int before = KFAST && rem < V ? V - rem : 0;
        base -= (int64_t)(int32_t)kstride * before;
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            const int last = KFAST ? rem - V : rem - 1;
            const int d = (kk(l) > last ? last - kk(l) : 0) + before;
            x[l] = gload_pack<R, PN>(base, voff[l] + (uint32_t)d * kstride + back);
        }
    }
    // multi-mode k: per-stage offsets from the table (k redirected to the last valid index); KFAST needs one entry
    static constexpr int NKO = KFAST ? 1 : NL;
    __device__ __forceinline__ void fetch_tab(uint32_t (&ko)[NKO], const uint32_t* tab, int64_t k0, int64_t kend) const {
#pragma unroll
        for (int l = 0; l < NKO; ++l) {
            const int64_t ki = k0 + kk(l), last = kend - (KFAST ? V : 1);
            ko[l] = tab[ki < last ? ki : last];
        }
    }
    __device__ __forceinline__ void load_tab(P (&x)[NL], gptr base, const uint32_t* tab, int64_t k0, int64_t kend) const {
        uint32_t ko[NKO];
        fetch_tab(ko, tab, k0, kend);
#pragma unroll
        for (int l = 0; l < NL; ++l) x[l] = gload_pack<R, PN>(base, voff[l] + ko[KFAST ? 0 : l]);
    }
    static_assert(V >= 1, "");
    // one load of a full stage (l is a compile-time constant at every call site)
    __device__ __forceinline__ void load_one(P (&x)[NL], int l, gptr base, const uint32_t (&ko)[NKO], bool tab) const {
        x[l] = gload_pack<R, PN>(base, voff[l] + (tab ? ko[KFAST ? 0 : l] : 0u));
    }
    // registers -> LDS tile [ROWS*RM][PITCH]; k past `rem` is zeroed when mask_tail.  A complex B (RM == 2) is
    // expanded to B'[2n][2k] = br, B'[2n][2k+1] = -bi, B'[2n+1][2k] = bi, B'[2n+1][2k+1] = br.
    static constexpr int VV = KFAST ? 1 : V;     // LDS stores per pass
    static constexpr int NSU = NP * VV;          // store units per thread and stage
    __device__ __forceinline__ void store(R* tile, const P (&x)[NL], bool mask_tail, int rem, bool conj) const {
#pragma unroll
        for (int u = 0; u < NSU; ++u) store_unit(tile, x, u, mask_tail, rem, conj);
    }
    // element e (possibly a run-time index, last stage only) of a load
    __device__ static __forceinline__ void pick(const P& src, int e, R& re, R& im) {
        re = src.v[0];
        im = EC == 2 ? src.v[EC - 1] : R(0);
#pragma unroll
        for (int i = 1; i < V; ++i) {
            re = e == i ? src.v[i * EC] : re;
            if (EC == 2) im = e == i ? src.v[i * EC + EC - 1] : im;
        }
    }
    // store unit u = (pass p, row v of the patch): one 16-byte (V > 1) or one-element LDS store (two for a complex B)
    __device__ __forceinline__ void store_unit(R* tile, const P (&x)[NL], int u, bool mask_tail, int rem, bool conj) const {
        const int p = u / VV, v = u % VV;
        // the thread's row and k position are recomputed from the thread index where they are needed (the last stage and
        // the element-wise path), so that they occupy no registers during the MFMA phase
        constexpr bool WHOLE = V * EC == C_::CH && (!KFAST || (RP * RM) % 32 == 0) && (KFAST || (KP & (KP - 1)) == 0);
        int t_ = 0;
        if (mask_tail || !WHOLE) {   // (not needed by a full stage of whole-chunk stores: nothing is emitted for those)
            t_ = threadIdx.x;
            asm volatile("" : "+v"(t_));
        }
        const int rq_ = KFAST ? t_ / KV : (t_ % RVN) * V, kq_ = KFAST ? (t_ % KV) * V : t_ / RVN;
        const int row = KFAST ? rq_ + p * RP : rq_ + v;
        const int kel0 = KFAST ? kq_ : (p * KP + kq_) * V;
        R out0[PN], out1[PN];
        // last stage: the window of a straddling vector was moved back by this many elements
        const int kshift = (mask_tail && KFAST && kel0 < rem && kel0 + V > rem) ? kel0 + V - rem : 0;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const P& src = x[KFAST ? p : p * V + j];
            const int e = KFAST ? j : v;
            const bool ok = !mask_tail || kel0 + j < rem;
            R sre, sim;
            if (mask_tail && V > 1) {
                pick(src, KFAST ? j + kshift : v + row_shift, sre, sim);   // indices past V-1 belong to masked k / rows outside the matrix
            } else {
                sre = src.v[EC * e];
                sim = EC == 2 ? src.v[EC * e + EC - 1] : R(0);
            }
            if constexpr (CX) {
                // conj and the minus sign of the expansion are one XOR of the sign bit each, with a mask that is uniform
                // and constant over the tile (a select between x and -x would cost two instructions per value)
                const R re = ok ? sre : R(0);
                const R im = ok ? flip_sign(sim, conj) : R(0);
                if constexpr (RM == 2) {
                    out0[2 * j] = re; out0[2 * j + 1] = ok ? flip_sign(sim, !conj) : R(0);
                    out1[2 * j] = im; out1[2 * j + 1] = re;
                } else {
                    out0[2 * j] = re; out0[2 * j + 1] = im;
                }
            } else {
                out0[j] = ok ? sre : R(0);
            }
        }
        // Whole-chunk stores derive their index from unit 0's with a constant or two, because the swizzle of a row only
        // depends on its low five bits: passes of a k-contiguous operand are RP * RM rows (a multiple of 32) apart; pass
        // p of a row-contiguous one is KP chunks further along k (kq < KP, a power of two: an XOR), and row v of its
        // patch is v * RM rows down with the chunk position XOR-ed by the same v * RM (rq is a multiple of V <= 4).
        int idx;
        if constexpr (WHOLE) {
            if constexpr (KFAST) idx = lds0 + p * RP * RM * C_::PITCH;
            else idx = ((lds0 ^ (v * RM * C_::CH)) + v * RM * C_::PITCH) ^ (p * KP * C_::CH);
        } else {
            idx = C_::lds_idx(row * RM, kel0 * EC);
        }
        lds_store_pack<R, PN>(tile + idx, out0);
        // the odd row below an even one: its swizzle differs in bit 0 only, i.e. the neighbouring chunk of the next row
        if constexpr (RM == 2) lds_store_pack<R, PN>(tile + (idx ^ C_::CH) + C_::PITCH, out1);
    }
};

// What one block works on: the problem (extents, operand bases, strides), its tile, batch entry and k split.
struct TileCtx {
    int64_t M, N, K;
    gptr Ap, Bp;
    void* Cp;
    Off32 am, ak, bk, bn;
    OffFn cm, cn;
    int tile_m, tile_n;
    int64_t batch;
    int split;
    bool grouped;   // a problem of a grouped launch: plain strided matrices, offsets relative to the problem's first element
};

template <class R, bool CX, bool AKF, bool BKF, int VA, int VB, int BNV = 128, int BMV = 128>
__device__ __forceinline__ void gemm128_body(const GemmArgs& g, const TileCtx& t, unsigned char* smem_raw) {
    typedef Cfg128<R, CX, BNV, BMV> C_;
    typedef typename Mfma<R>::acc_t acc_t;
    constexpr int BM = C_::BM, BN = C_::BN, BKE = C_::BKE, PITCH = C_::PITCH, BNE = C_::BNE, CH = C_::CH;
    constexpr int TM = C_::TM, TN = C_::TN;
    R* As = reinterpret_cast<R*>(smem_raw);   // [2][BM][PITCH]
    R* Bs = As + 2 * BM * PITCH;              // [2][BN][PITCH]

    const int64_t M = t.M, N = t.N, K = t.K;
    gptr Ap = t.Ap, Bp = t.Bp;
    void* Cp = t.Cp;
    const Off32 am = t.am, ak = t.ak, bk = t.bk, bn = t.bn;
    const OffFn cm = t.cm, cn = t.cn;
    const int tile_m = t.tile_m, tile_n = t.tile_n;
    const int64_t batch = t.batch;
    const int split = t.split;
    const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BNE;
    const int64_t kbeg = (int64_t)split * g.k_per_split;
    const int64_t kend = (g.nsplit > 1 && kbeg + g.k_per_split < K) ? kbeg + g.k_per_split : K;
    const int rowsA = (int)(M - m0 < BM ? M - m0 : BM), rowsB = (int)(N - n0 < BNE ? N - n0 : BNE);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    typedef OperandMap<R, CX, BM, AKF, VA, 1, BNV> MapA;
    typedef OperandMap<R, CX, BNE, BKF, VB, (CX ? 2 : 1), BNV> MapB;
    MapA ma;
    MapB mb;
    // single-stride rows: the tile's first row goes into the 64-bit base and the offsets start at row 0, so that they
    // span one tile whatever the operand's size.  A vector moved back at a matrix edge can start a few rows before
    // the tile: the host's bias leaves room for that.  Grouped problems carry no bias (and are small): their offsets
    // stay relative to the problem's first row.
    const bool rebase_a = !am.tab && !t.grouped, rebase_b = !bn.tab && !t.grouped;
    if (rebase_a) Ap += (int64_t)(int32_t)am.stride * m0;
    if (rebase_b) Bp += (int64_t)(int32_t)bn.stride * n0;
    ma.init(am, ak, rebase_a ? 0 : m0, rowsA);
#pragma unroll
    for (int l = 0; l < MapA::NL; ++l) ma.voff[l] += t.grouped ? 0u : g.bias_a32;
    mb.init(bn, bk, rebase_b ? 0 : n0, rowsB);
#pragma unroll
    for (int l = 0; l < MapB::NL; ++l) mb.voff[l] += t.grouped ? 0u : g.bias_b32;
    // uniform bases; single-stride k advances them by one stage per iteration
    gptr sa = Ap + (ak.tab ? 0 : (int64_t)(int32_t)ak.stride * kbeg);
    gptr sb = Bp + (bk.tab ? 0 : (int64_t)(int32_t)bk.stride * kbeg);
    const int64_t stepA = ak.tab ? 0 : (int64_t)(int32_t)ak.stride * BKE;
    const int64_t stepB = bk.tab ? 0 : (int64_t)(int32_t)bk.stride * BKE;

    const int wm0 = (wave / C_::WAVES_N) * C_::WM, wn0 = (wave % C_::WAVES_N) * C_::WN;
    const int lrow = lane & 15, lgrp = lane >> 4;
    // chunk swizzle of the fragment rows: block i of the wave is rows w0 + 16 i + lrow with w0 a multiple of 32, so bits
    // 0-3 of the row are lrow's and bit 4 is that of (w0 >> 4) + i
    const int swl = (lrow & 7) ^ (lrow >> 3);
    const int swa0 = (wm0 >> 4) & 1, swb0 = (wn0 >> 4) & 1;

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t{0, 0, 0, 0};

    typename MapA::P va[MapA::NL];
    typename MapB::P vb[MapB::NL];
    const int64_t klen = kend > kbeg ? kend - kbeg : 0;
    const int64_t nstage = (klen + BKE - 1) / BKE;
    const int rem = (int)(klen - (nstage - 1) * BKE);   // k elements in the last stage (1..BKE)
    const bool ktab = ak.tab != nullptr;               // the host builds k tables for both operands or for none
    // the last stage is a full one and no 16-byte access straddles the matrix edge: it is stored like any other
    const bool plain_last = rem == BKE && (AKF || VA == 1 || rowsA % VA == 0) && (BKF || VB == 1 || rowsB % VB == 0);

    auto load_fast = [&]() {
        sa = uniform_ptr(sa);
        sb = uniform_ptr(sb);
        ma.load_fast(va, sa);
        mb.load_fast(vb, sb);
        sa += stepA;
        sb += stepB;
    };
    auto load_tail = [&]() {
        ma.load_tail(va, sa, rem, ak.stride, am.stride);
        mb.load_tail(vb, sb, rem, bk.stride, bn.stride);
    };
    auto load_tab = [&](int64_t s) {
        ma.load_tab(va, sa, ak.tab, kbeg + s * BKE, kend);
        mb.load_tab(vb, sb, bk.tab, kbeg + s * BKE, kend);
    };
    auto store_stage = [&](int buf, bool mask_tail) {
        ma.store(As + buf * BM * PITCH, va, mask_tail, rem, g.conj_a != 0);
        mb.store(Bs + buf * BN * PITCH, vb, mask_tail, rem, g.conj_b != 0);
    };

    typedef typename RawVec<R, CH>::type Chunk;
    auto compute = [&](int buf) {
        const R* as = As + buf * BM * PITCH + (wm0 + lrow) * PITCH;
        const R* bs = Bs + buf * BN * PITCH + (wn0 + lrow) * PITCH;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            Chunk a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const Chunk*>(as + i * 16 * PITCH + ((2 * lgrp + h) ^ swl ^ (((swa0 + i) & 1) << 1)) * CH);
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = *reinterpret_cast<const Chunk*>(bs + j * 16 * PITCH + ((2 * lgrp + h) ^ swl ^ (((swb0 + j) & 1) << 1)) * CH);
#pragma unroll
            for (int c = 0; c < CH; ++c)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<R>::run(a[i][c], b[j][c], acc[i][j]);
        }
    };

    // One full iteration of the main loop with everything else issued in the shadow of the MFMAs: the global loads
    // of stage s+1 go out between the MFMAs of the first half of stage s, the LDS stores of stage s+1 (into the other
    // buffer, which nobody reads during this iteration) between those of the second half.  An MFMA occupies the matrix core for 32 or 64 cycles after it issues, so the instructions placed
    // between two of them cost nothing as long as they take less than that to issue.  sched_barrier pins the
    // order against the compiler.  With multi-mode k the table entries of stage s+2 are fetched one iteration
    // ahead, so no load waits for its offset.
    constexpr int HALF = TM * TN * CH;                        // MFMAs per half stage
    constexpr int NLD = MapA::NL + MapB::NL, NST = MapA::NSU + MapB::NSU;
    // spread evenly over the half stage (measured: better than bunching the loads early and the stores late)
    constexpr int LD_EVERY = HALF / (NLD + 1) > 0 ? HALF / (NLD + 1) : 1;
    constexpr int ST_EVERY = HALF / (NST + 1) > 0 ? HALF / (NST + 1) : 1;
    constexpr int ST_FIRST = 0;
    static_assert(LD_EVERY * NLD <= HALF && ST_FIRST + ST_EVERY * NST <= HALF, "one half stage must take all loads / stores");
    uint32_t ka[MapA::NKO], kb[MapB::NKO];   // multi-mode k: table entries of the stage whose loads are issued next
    auto stage_interleaved = [&](int buf, bool tab, int64_t k0_after_next) {
        const R* as = As + buf * BM * PITCH + (wm0 + lrow) * PITCH;
        const R* bs = Bs + buf * BN * PITCH + (wn0 + lrow) * PITCH;
        R* as_next = As + (buf ^ 1) * BM * PITCH;
        R* bs_next = Bs + (buf ^ 1) * BN * PITCH;
        Chunk a[2][TM], b[2][TN];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < TM; ++i) a[h][i] = *reinterpret_cast<const Chunk*>(as + i * 16 * PITCH + ((2 * lgrp + h) ^ swl ^ (((swa0 + i) & 1) << 1)) * CH);
#pragma unroll
            for (int j = 0; j < TN; ++j) b[h][j] = *reinterpret_cast<const Chunk*>(bs + j * 16 * PITCH + ((2 * lgrp + h) ^ swl ^ (((swb0 + j) & 1) << 1)) * CH);
        }
        if (!tab) {
            sa = uniform_ptr(sa);
            sb = uniform_ptr(sb);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    acc[i][j] = Mfma<R>::run(a[0][i][c], b[0][j][c], acc[i][j]);
                    const int m = (c * TM + i) * TN + j;
                    if (m % LD_EVERY == LD_EVERY - 1 && m / LD_EVERY < NLD) {
                        const int l = m / LD_EVERY;
                        if (l < MapA::NL) ma.load_one(va, l, sa, ka, tab);
                        else mb.load_one(vb, l - MapA::NL, sb, kb, tab);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
        if (tab) {
            ma.fetch_tab(ka, ak.tab, k0_after_next, kend);
            mb.fetch_tab(kb, bk.tab, k0_after_next, kend);
        } else {
            sa += stepA;
            sb += stepB;
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < CH; ++c)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    acc[i][j] = Mfma<R>::run(a[1][i][c], b[1][j][c], acc[i][j]);
                    const int m = (c * TM + i) * TN + j;
                    if (m >= ST_FIRST && (m - ST_FIRST) % ST_EVERY == ST_EVERY - 1 && (m - ST_FIRST) / ST_EVERY < NST) {
                        const int u = (m - ST_FIRST) / ST_EVERY;
                        if (u < MapA::NSU) ma.store_unit(as_next, va, u, false, rem, g.conj_a != 0);
                        else mb.store_unit(bs_next, vb, u - MapA::NSU, false, rem, g.conj_b != 0);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
    };

    if (nstage > 0) {
        // prologue: stage 0 into buffer 0 and, when a full stage follows, its loads into the registers
        if (nstage == 1) {
            if (ktab) load_tab(0);
            else if (plain_last) load_fast();
            else load_tail();
        } else {
            if (ktab) load_tab(0);
            else load_fast();
        }
        // (two calls: with the flag a constant, the store of a full stage carries none of the masking arithmetic)
        if (nstage == 1 && !plain_last) store_stage(0, true);
        else store_stage(0, false);
        if (ktab) {
            ma.fetch_tab(ka, ak.tab, kbeg + BKE, kend);
            mb.fetch_tab(kb, bk.tab, kbeg + BKE, kend);
        }
        __syncthreads();
        int64_t s = 0;
        for (; s + 2 < nstage; ++s) {
            // Two blocks share a CU.  The arbiter favours the older wave, so one block runs ahead and the other is
            // left to finish alone; when all blocks of a launch start together and nothing follows them, lowering a
            // block's issue priority as it progresses keeps the one that is behind ahead in the arbitration, and the
            // two finish together (config 1: 1 % faster).  With more tiles than resident blocks it is the other way
            // round: blocks that end at different times overlap their epilogues and prologues with their neighbours'
            // main loops, so nothing is done to align them (the grouped launch of config 4 lost 1.5 % to this).
            if (g.one_round && (s & 3) == 0) {
                const int q = (int)((4 * s) / nstage);
                if (q == 0) __builtin_amdgcn_s_setprio(3);
                else if (q == 1) __builtin_amdgcn_s_setprio(2);
                else if (q == 2) __builtin_amdgcn_s_setprio(1);
                else __builtin_amdgcn_s_setprio(0);
            }
            stage_interleaved((int)(s & 1), ktab, kbeg + (s + 2) * BKE);
            __syncthreads();
        }
        if (s + 1 < nstage) {
            if (ktab) load_tab(s + 1);
            else if (plain_last) load_fast();
            else load_tail();
            compute((int)(s & 1));
            if (plain_last) store_stage((int)((s + 1) & 1), false);
            else store_stage((int)((s + 1) & 1), true);
            __syncthreads();
            ++s;
        }
        compute((int)(s & 1));
    }

    // ---- epilogue: real column wn0 + 16 j + lrow; for complex, column 2n+p is part p of element n ----------
    const int64_t NR = CX ? 2 * N : N;
    const int64_t n0r = CX ? 2 * n0 : n0;
    // A tile that lies wholly inside the matrix (all but the last row and column of tiles) is written without a
    // bounds predicate per element: one address per accumulator row, the four column blocks at constant offsets from it.
    const bool full_tile = m0 + BM <= M && n0r + BN <= NR;
    if (g.nsplit > 1) {
        R* P = reinterpret_cast<R*>(g.partial) + ((int64_t)split * g.nbatch + batch) * M * NR;
        if (full_tile) {
            R* p0 = P + (m0 + wm0) * NR + n0r + wn0 + lrow;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    R* p = p0 + (int64_t)(16 * i + Mfma<R>::row(lane, r)) * NR;
#pragma unroll
                    for (int j = 0; j < TN; ++j) p[16 * j] = acc[i][j][r];
                }
            return;
        }
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
    R* Cb = reinterpret_cast<R*>(Cp) + (t.grouped ? 0 : off_of(g.cb, batch)) * (CX ? 2 : 1);
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    const bool real_scalars = g.alpha_im == 0.0 && g.beta_im == 0.0;
    // C contiguous along n (the usual case; the host exchanges the operands to get it), real scalars: the same for the result
    if (full_tile && !cn.tab && cn.stride == 1 && (!CX || real_scalars)) {
        R* c0 = Cb + n0r + wn0 + lrow;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                R* p = c0 + off_of(cm, m0 + wm0 + 16 * i + Mfma<R>::row(lane, r)) * (CX ? 2 : 1);
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    R out = ar * acc[i][j][r];
                    if (g.use_beta) out += br * p[16 * j];
                    p[16 * j] = out;
                }
            }
        return;
    }
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
                    if (real_scalars) {   // real alpha and beta act on the two parts separately: no exchange
                        if (ok) {
                            R out = ar * v;
                            if (g.use_beta) out += br * *dst;
                            *dst = out;
                        }
                        continue;
                    }
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

// One tile of a uniform launch (single problem, batched, split-K) or of a grouped launch whose tiles all have this shape.
template <class R, bool CX, bool AKF, bool BKF, int VA, int VB, int BNV = 128, int BMV = 128>
__global__ void __launch_bounds__((Cfg128<R, CX, BNV, BMV>::NT), (Cfg128<R, CX, BNV, BMV>::MIN_WAVES)) gemm128_kernel(GemmArgs g) {
    typedef typename ElemT<R, CX>::type E;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    TileCtx t;
    t.M = g.M; t.N = g.N; t.K = g.K;
    t.Ap = as_global(g.A32);
    t.Bp = as_global(g.B32);
    t.Cp = g.C;
    t.am = g.am32; t.ak = g.ak32; t.bk = g.bk32; t.bn = g.bn32;
    t.cm = g.cm; t.cn = g.cn;
    t.batch = 0;
    t.split = 0;
    t.grouped = g.problems != nullptr;
    if (g.problems) {
        const int4 tm = g.tile_map[blockIdx.x];
        const GroupProblem& p = g.problems[tm.x];
        t.M = p.M; t.N = p.N; t.K = p.K;
        t.Ap = as_global(p.A); t.Bp = as_global(p.B); t.Cp = p.C;
        t.am.stride = (uint32_t)(p.sam * (int64_t)sizeof(E)); t.ak.stride = (uint32_t)(p.sak * (int64_t)sizeof(E));
        t.bk.stride = (uint32_t)(p.sbk * (int64_t)sizeof(E)); t.bn.stride = (uint32_t)(p.sbn * (int64_t)sizeof(E));
        t.cm.stride = p.scm; t.cn.stride = p.scn;
        t.tile_m = tm.y;
        t.tile_n = tm.z;
    } else {
        // one-dimensional grid: tiles of one (batch, split) pair are adjacent logical positions
        const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n;
        const uint64_t lb = logical_block(blockIdx.x, gridDim.x);
        const uint32_t lz = (uint32_t)(lb / tiles);
        tile_of((uint32_t)(lb % tiles), g.tiles_m, g.tiles_n, t.tile_m, t.tile_n);
        t.split = (int)(lz % (uint32_t)g.nsplit);
        t.batch = lz / (uint32_t)g.nsplit;
        t.Ap += off_of(g.ab, t.batch) * (int64_t)sizeof(E);
        t.Bp += off_of(g.bb, t.batch) * (int64_t)sizeof(E);
    }
    gemm128_body<R, CX, AKF, BKF, VA, VB, BNV, BMV>(g, t, smem_raw);
}

// Grouped launch with a tile shape per map entry (tile_map[].w): 0 = 128 x 128; 1 = 128 rows x 64 real columns (a last
// column strip of at most 64); 2 = 64 rows x 128 real columns (a last row strip of at most 64), computed as the transposed
// product with the operands exchanged, so that the strip is again the thin right-hand side; -1 = no tile (padding that
// keeps the per-XCD lists of the map equally long).  The branch is uniform over the block; the three bodies never run
// in the same block, so registers and LDS are those of the largest.
template <class R, bool CX, bool AKF, bool BKF, int V>
__global__ void __launch_bounds__((Cfg128<R, CX, 128>::NT), (Cfg128<R, CX, 128>::MIN_WAVES)) gemm128_grouped_kernel(GemmArgs g) {
    typedef typename ElemT<R, CX>::type E;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int4 tm = g.tile_map[blockIdx.x];
    if (tm.x < 0) return;
    const GroupProblem& p = g.problems[tm.x];
    const int kind = __builtin_amdgcn_readfirstlane(tm.w);
    TileCtx t;
    t.batch = 0;
    t.split = 0;
    t.grouped = true;
    t.tile_m = tm.y;
    t.tile_n = tm.z;
    t.K = p.K;
    t.Cp = p.C;
    t.am.tab = t.ak.tab = t.bk.tab = t.bn.tab = nullptr;
    t.cm.tab = t.cn.tab = nullptr;
    constexpr int64_t EB = (int64_t)sizeof(E);
    // a row-contiguous B of 4-byte reals has more threads than 16-byte accesses over 64 columns: 8-byte accesses there
    constexpr int VTHIN = (V > 1 && sizeof(R) == 4) ? V / 2 : V;
    if (kind != 2) {
        t.M = p.M; t.N = p.N;
        t.Ap = as_global(p.A); t.Bp = as_global(p.B);
        t.am.stride = (uint32_t)(p.sam * EB); t.ak.stride = (uint32_t)(p.sak * EB);
        t.bk.stride = (uint32_t)(p.sbk * EB); t.bn.stride = (uint32_t)(p.sbn * EB);
        t.cm.stride = p.scm; t.cn.stride = p.scn;
        if (kind == 0) gemm128_body<R, CX, AKF, BKF, V, V, 128>(g, t, smem_raw);
        else gemm128_body<R, CX, AKF, BKF, V, (BKF ? V : VTHIN), 64>(g, t, smem_raw);
    } else {
        // C^T = B^T A^T: the body's A is B seen with rows n, its B is A seen with columns m
        t.M = p.N; t.N = p.M;
        t.Ap = as_global(p.B); t.Bp = as_global(p.A);
        t.am.stride = (uint32_t)(p.sbn * EB); t.ak.stride = (uint32_t)(p.sbk * EB);
        t.bk.stride = (uint32_t)(p.sak * EB); t.bn.stride = (uint32_t)(p.sam * EB);
        t.cm.stride = p.scn; t.cn.stride = p.scm;
        gemm128_body<R, CX, BKF, AKF, V, (AKF ? V : VTHIN), 64>(g, t, smem_raw);
    }
}

template <class R, bool CX, bool AKF, bool BKF, int VA, int VB, int BNV = 128, int BMV = 128>
inline void launch_gemm128_variant(const GemmArgs& g, dim3 grid, hipStream_t st) {
    static bool once = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm128_kernel<R, CX, AKF, BKF, VA, VB, BNV, BMV>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)Cfg128<R, CX, BNV, BMV>::LDS_BYTES);
        return true;
    }();
    (void)once;
    typedef Cfg128<R, CX, BNV, BMV> C_;
    const size_t lds = C_::LDS_BYTES;
    const dim3 block(C_::NT);
    TFH_LAUNCH_TIMED((gemm128_kernel<R, CX, AKF, BKF, VA, VB, BNV, BMV>), grid, block, lds, st, g);
    if (BMV == 64) note_kernel("(gemm128_kernel, 64x64 tiles)");
    else if (BNV == 64) note_kernel("(gemm128_kernel, 128x64 tiles)");
}

template <class R, bool CX, int V, int BNV = 128>
inline void launch_gemm128_layout(const GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    if (akf) {
        if (bkf) launch_gemm128_variant<R, CX, true, true, V, V, BNV>(g, grid, st);
        else launch_gemm128_variant<R, CX, true, false, V, V, BNV>(g, grid, st);
    } else {
        if (bkf) launch_gemm128_variant<R, CX, false, true, V, V, BNV>(g, grid, st);
        else launch_gemm128_variant<R, CX, false, false, V, V, BNV>(g, grid, st);
    }
}

// g.vec: both operands satisfy the alignment and divisibility rules of 16-byte accesses
template <class R, bool CX>
inline void launch_gemm128_any(const GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    constexpr int VMAX = Cfg128<R, CX>::VMAX;
    if constexpr (VMAX > 1) {
        if (g.vec) {
            launch_gemm128_layout<R, CX, VMAX>(g, grid, akf, bkf, st);
            return;
        }
    }
    launch_gemm128_layout<R, CX, 1>(g, grid, akf, bkf, st);
}

// Grouped launch with per-tile shapes (16-byte accesses only: g.vec; the scalar-access fallback keeps uniform tiles).
template <class R, bool CX, bool AKF, bool BKF>
inline void launch_gemm128_grouped_variant(const GemmArgs& g, dim3 grid, hipStream_t st) {
    constexpr int V = Cfg128<R, CX>::VMAX;
    static bool once = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm128_grouped_kernel<R, CX, AKF, BKF, V>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)Cfg128<R, CX, 128>::LDS_BYTES);
        return true;
    }();
    (void)once;
    typedef Cfg128<R, CX, 128> C_;
    const size_t lds = C_::LDS_BYTES;
    const dim3 block(C_::NT);
    TFH_LAUNCH_TIMED((gemm128_grouped_kernel<R, CX, AKF, BKF, V>), grid, block, lds, st, g);
}
template <class R, bool CX>
inline void launch_gemm128_grouped_any(const GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    if (akf) {
        if (bkf) launch_gemm128_grouped_variant<R, CX, true, true>(g, grid, st);
        else launch_gemm128_grouped_variant<R, CX, true, false>(g, grid, st);
    } else {
        if (bkf) launch_gemm128_grouped_variant<R, CX, false, true>(g, grid, st);
        else launch_gemm128_grouped_variant<R, CX, false, false>(g, grid, st);
    }
}

// 128 x 64 tiles for a thin right-hand side.  A row-contiguous B of f32 / complex64 has more threads than 16-byte
// accesses over 64 columns give work to: that loader uses 8-byte accesses (two f32, one complex64).
template <class R, bool CX>
inline void launch_gemm128x64_any(const GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    constexpr int VMAX = Cfg128<R, CX>::VMAX;
    if constexpr (VMAX > 1) {
        if (g.vec) {
            if constexpr (sizeof(R) == 8) {
                launch_gemm128_layout<R, CX, VMAX, 64>(g, grid, akf, bkf, st);
            } else {
                constexpr int VBR = VMAX / 2;
                if (bkf) {
                    if (akf) launch_gemm128_variant<R, CX, true, true, VMAX, VMAX, 64>(g, grid, st);
                    else launch_gemm128_variant<R, CX, false, true, VMAX, VMAX, 64>(g, grid, st);
                } else {
                    if (akf) launch_gemm128_variant<R, CX, true, false, VMAX, VBR, 64>(g, grid, st);
                    else launch_gemm128_variant<R, CX, false, false, VMAX, VBR, 64>(g, grid, st);
                }
            }
            return;
        }
    }
    launch_gemm128_layout<R, CX, 1, 64>(g, grid, akf, bkf, st);
}

// 64 x 64 tiles.  A row-contiguous operand of 4-byte reals over 64 rows is loaded with 8-byte accesses (as the thin B above).
template <class R, bool CX>
inline void launch_gemm64x64_any(const GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st) {
    constexpr int VMAX = Cfg128<R, CX>::VMAX;
    if constexpr (VMAX > 1) {
        if (g.vec) {
            constexpr int VR = sizeof(R) == 8 ? VMAX : VMAX / 2;   // row-contiguous operand
            if (akf) {
                if (bkf) launch_gemm128_variant<R, CX, true, true, VMAX, VMAX, 64, 64>(g, grid, st);
                else launch_gemm128_variant<R, CX, true, false, VMAX, VR, 64, 64>(g, grid, st);
            } else {
                if (bkf) launch_gemm128_variant<R, CX, false, true, VR, VMAX, 64, 64>(g, grid, st);
                else launch_gemm128_variant<R, CX, false, false, VR, VR, 64, 64>(g, grid, st);
            }
            return;
        }
    }
    if (akf) {
        if (bkf) launch_gemm128_variant<R, CX, true, true, 1, 1, 64, 64>(g, grid, st);
        else launch_gemm128_variant<R, CX, true, false, 1, 1, 64, 64>(g, grid, st);
    } else {
        if (bkf) launch_gemm128_variant<R, CX, false, true, 1, 1, 64, 64>(g, grid, st);
        else launch_gemm128_variant<R, CX, false, false, 1, 1, 64, 64>(g, grid, st);
    }
}

}  // namespace gemm

// One translation unit per dtype instantiates its four layout variants.
void launch_gemm128_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_f64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_c64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
// ... and the same layouts with 128 x 64 tiles
void launch_gemm128x64_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128x64_f64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128x64_c64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128x64_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
// ... with 64 x 64 tiles (translation units of their own)
void launch_gemm64x64_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm64x64_f64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm64x64_c64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm64x64_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
// ... and the grouped kernel with a tile shape per map entry
void launch_gemm128_grouped_f32(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_grouped_f64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_grouped_c64(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);
void launch_gemm128_grouped_c128(const gemm::GemmArgs& g, dim3 grid, bool akf, bool bkf, hipStream_t st);

}  // namespace tfh
