// k_gemm_bfirst.hip -- batched products whose batch index is the contiguous one in all three tensors:
// column-major "bij,bjk->bik", the layout of every batched example in tenferro-einsum/src/lib.rs:74-93
// (MemoryOrder::ColumnMajor, tenferro-tensor/src/lib.rs:110-127), through PrimDescriptor::Contract /
// BatchedGemm (tenferro-prims/src/lib.rs:156-168, 227-239).
//
// In that layout neither the rows nor the k of one batch entry are contiguous: the 128-byte line at (row, k) holds
// that element of 8 (complex128), 16 (f64, complex64) or 32 (f32) consecutive batch entries.  A tile kernel that
// works on one batch entry at a time would use 8 or 16 bytes of every line it fetches.  Here a block takes ALL the
// batch entries of a line at once: its tile is NB batch entries x 32 rows x 32 columns, a stage is four k of it.
//
//   loads : thread t moves 16 bytes (chunk c = t % 8 of a line) of line (row t / 8, k p) in pass p = 0..3, for A and
//           for B: every load instruction of a wave covers eight whole lines.
//   LDS   : the lines are kept as they are, line j = k * 32 + row at byte j * 128, chunk c at position
//           c ^ f(j), f(j) = (j ^ (j >> 3)) & 7 -- a store of eight lanes covers one line's 128 bytes, and the sixteen
//           lanes that a 16-byte fragment read serves together (rows 0-7 of one k with rows 8-15 of the next)
//           touch sixteen different 16-byte bank groups.
//   MFMAs : wave w owns chunks 2w and 2w+1 of every line, i.e. 2 (complex128), 4 (f64, complex64) or 8 (f32) batch
//           entries, and computes their 32 x 32 tiles with 16x16x4 MFMAs: a fragment read of 16 bytes at
//           (row lane % 16, k lane / 16) IS the MFMA operand of all the batch entries in the chunk.  Complex
//           products run as real ones on A' = [re, im] along k and B' = [[br, bi], [-bi, br]]: a lane picks the
//           part it needs (and its sign) when it reads the fragment; conj is a sign flip when the line is stored.
//   C     : a lane holds, for its (row, column), the results of its wave's batch entries only; the tile goes through LDS
//           once more so that eight lanes store one whole 128-byte line of C.
//
// Two blocks share a CU (64 KB of LDS and at most 256 VGPRs each).
#include <algorithm>
#include <cstring>
#include <vector>

#include "gemm128.hpp"


namespace tfh {
namespace gemm {


template <class R, bool CX>
struct BfCfg {
    static constexpr int EC = CX ? 2 : 1;
    static constexpr int EB = (int)sizeof(R) * EC;      // bytes per element
    static constexpr int EPC = 16 / EB;                 // batch entries per 16-byte chunk
    static constexpr int NB = 8 * EPC;                  // batch entries per block: one 128-byte line
    static constexpr int WB = 2 * EPC;                  // batch entries per wave: two chunks
    static constexpr int T = 32;                        // rows and element columns per tile
    static constexpr int KL = 4;                        // elements of k per stage (one line each)
    static constexpr int KSTEPS = CX ? 2 : 1;           // MFMA k steps per stage
    static constexpr int NJ = CX ? 4 : 2;               // 16-wide real column blocks per tile
    static constexpr int OPER_BYTES = KL * T * 128;     // one operand's stage: 16 KB
    static constexpr int STAGE_BYTES = 2 * OPER_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;   // double-buffered: 64 KB
    static constexpr int RPC = 16 / (int)sizeof(R);     // reals per chunk
};

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
template <int ALIGN> struct U4U;
template <> struct U4U<4> { typedef uint32_t type __attribute__((ext_vector_type(4), aligned(4))); };
template <> struct U4U<8> { typedef uint32_t type __attribute__((ext_vector_type(4), aligned(8))); };

template <class R, bool CX, int D>
__global__ void __launch_bounds__(256, 2) gemm_bfirst_kernel(BfArgs g) {
    typedef BfCfg<R, CX> C_;
    typedef typename Mfma<R>::acc_t acc_t;
    typedef typename RawVec<R, C_::RPC>::type Chunk;
    constexpr int EB = C_::EB, EPC = C_::EPC, NB = C_::NB, WB = C_::WB, T = C_::T, KL = C_::KL, NJ = C_::NJ;
    constexpr int OPER = C_::OPER_BYTES, STAGE = C_::STAGE_BYTES;
    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane & 15, lgrp = lane >> 4;

    // block -> (outer batch entry, group of NB batch entries, tile): the tiles of one group are adjacent logical
    // positions, which one XCD works through at about the same time, so the A rows and B columns they share meet
    // in that L2
    const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n;
    const uint64_t lb = logical_block(blockIdx.x, gridDim.x);
    const uint32_t tile = (uint32_t)(lb % tiles);
    const uint64_t gi = lb / tiles;
    const int64_t grp = (int64_t)(gi % (uint32_t)g.groups), ob = (int64_t)(gi / (uint32_t)g.groups);
    const int tile_m = (int)(tile % (uint32_t)g.tiles_m), tile_n = (int)(tile / (uint32_t)g.tiles_m);
    const int64_t m0 = (int64_t)tile_m * T, n0 = (int64_t)tile_n * T, b0 = grp * NB;
    const int rowsA = (int)(g.M - m0 < T ? g.M - m0 : T), rowsB = (int)(g.N - n0 < T ? g.N - n0 : T);
    const int chunks_valid = (int)((g.nb - b0) / EPC < 8 ? (g.nb - b0) / EPC : 8);   // whole chunks of this group

    // ---- loader: chunk c of line (row lr, k p) in pass p; rows, and chunks, past the edge are redirected to valid ones
    // (their products belong to rows, columns or batch entries that are never stored)
    const int c = tid & 7, lr = tid >> 3;
    const int cc = c < chunks_valid ? c : 0;
    const int ra_ = lr < rowsA ? lr : rowsA - 1, rb_ = lr < rowsB ? lr : rowsB - 1;
    const uint32_t voa = (uint32_t)(((int64_t)ra_ * g.sam + (int64_t)cc * EPC) * EB);
    const uint32_t vob = (uint32_t)(((int64_t)rb_ * g.sbn + (int64_t)cc * EPC) * EB);
    gptr sa = as_global(g.A) + (ob * g.sao + b0 + m0 * g.sam) * EB;
    gptr sb = as_global(g.B) + (ob * g.sbo + b0 + n0 * g.sbn) * EB;
    const int64_t stepA = g.sak * EB, stepB = g.sbk * EB;
    const uint32_t wofs = (uint32_t)(lr * 128 + ((c ^ (lr & 7) ^ (lr >> 3)) << 4));
    // conj: the sign bit of the imaginary parts of a chunk, flipped when the line is stored
    u4 cja = u4{0, 0, 0, 0}, cjb = u4{0, 0, 0, 0};
    if constexpr (CX) {
        const u4 m = sizeof(R) == 8 ? u4{0, 0, 0, 0x80000000u} : u4{0, 0x80000000u, 0, 0x80000000u};
        if (g.conj_a) cja = m;
        if (g.conj_b) cjb = m;
    }

    // ---- fragment addresses (bytes inside one operand's stage; see the layout note above)
    uint32_t fa, fb;       // A and B: XOR-ed with 16 * (q ^ ...) and offset by constants per block
    R bsign = R(0);        // complex B': -bi for (k part 1, column part 0): a sign mask applied to the fragment
    uint32_t bmask_hi = 0;
    if constexpr (!CX) {
        fa = (uint32_t)(lgrp * 4096 + lrow * 128 + (((2 * wave) ^ (lrow & 7) ^ (lrow >> 3) ^ (4 * (lgrp & 1))) << 4));
        fb = fa;
    } else {
        fa = (uint32_t)((lgrp >> 1) * 4096 + lrow * 128 + (((2 * wave) ^ (lrow & 7) ^ (lrow >> 3) ^ (4 * (lgrp >> 1))) << 4) +
                        (lgrp & 1) * (int)sizeof(R));
        fb = (uint32_t)((lgrp >> 1) * 4096 + (lrow >> 1) * 128 + (((2 * wave) ^ (lrow >> 1) ^ (4 * (lgrp >> 1))) << 4) +
                        (((lgrp & 1) != (lrow & 1)) ? (int)sizeof(R) : 0));
        bmask_hi = ((lgrp & 1) == 1 && (lrow & 1) == 0) ? 0x80000000u : 0u;
    }
    (void)bsign;

    acc_t acc[WB][2][NJ];
#pragma unroll
    for (int w_ = 0; w_ < WB; ++w_)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < NJ; ++j) acc[w_][i][j] = acc_t{0, 0, 0, 0};

    typedef const __attribute__((address_space(1))) typename U4U<(int)sizeof(R)>::type* gu4;
    // D stages on their way from global memory to LDS, each in a register set of its own (A passes, then B passes): a
    // stage of 16 or 32 MFMAs per wave is shorter than the memory latency
    u4 stg[D][2 * KL];
    const int K = (int)g.K;
    const int nstage = (K + KL - 1) / KL;

    // The sum over k may run in any order: stage 0 takes the K % KL lines left over (KL when there are none), so that every
    // later stage is a full one: rem0 lines at k = 0, stage t >= 1 at k = rem0 + (t - 1) * KL.  A k past the end (stage 0's
    // missing lines, stages past the last that the loop still loads) is redirected to a valid k.  All of this is scalar
    // arithmetic that stays out of the loop: the load stream has one uniform pointer per operand (the first line of the
    // stage that is loaded next), advanced by one stage per iteration until it stands on the last stage, and the four lines
    // of a stage lie at loop-invariant offsets from it.
    const int rem0 = K - (nstage - 1) * KL;
    int64_t off0A[KL], off0B[KL], offA[KL], offB[KL];
#pragma unroll
    for (int p = 0; p < KL; ++p) {
        const int p0 = p < rem0 ? p : rem0 - 1, p1 = nstage > 1 ? p : p0;
        off0A[p] = p0 * stepA; off0B[p] = p0 * stepB;
        offA[p] = p1 * stepA; offB[p] = p1 * stepB;
    }
    gptr ldA = sa + (nstage > 1 ? rem0 : 0) * stepA, ldB_ = sb + (nstage > 1 ? rem0 : 0) * stepB;   // stage 1
    int l_stage = 1;
    const int64_t stepKA = KL * stepA, stepKB = KL * stepB;
    auto advance_loads = [&]() __attribute__((always_inline)) {
        const bool more = l_stage < nstage - 1;
        ldA += more ? stepKA : 0;
        ldB_ += more ? stepKB : 0;
        ++l_stage;
    };
    // load unit u of the stage the load stream stands on (first: of stage 0): pass u of A (u < KL) or pass u - KL of B
    auto load_unit = [&](u4 (&x)[2 * KL], int u, bool first) __attribute__((always_inline)) {
        const int p = u % KL;
        if (u < KL) x[u] = __builtin_nontemporal_load(reinterpret_cast<gu4>(uniform_ptr(first ? sa + off0A[p] : ldA + offA[p]) + voa));
        else x[u] = __builtin_nontemporal_load(reinterpret_cast<gu4>(uniform_ptr(first ? sb + off0B[p] : ldB_ + offB[p]) + vob));
    };
    // store unit u of a stage: pass u of A (u < KL) or pass u - KL of B; stage 0's missing lines are zeros
    auto store_unit = [&](int buf, const u4 (&x)[2 * KL], int u, bool first) __attribute__((always_inline)) {
        const int p = u % KL;
        u4 v = x[u] ^ (u < KL ? cja : cjb);
        if (first && p >= rem0) v = u4{0, 0, 0, 0};
        const uint32_t o = (wofs ^ (uint32_t)((p & 1) << 6)) + (uint32_t)(p * 4096 + (u < KL ? 0 : OPER));
        *reinterpret_cast<u4*>(smem + buf * STAGE + o) = v;
    };
    // A stage is multiplied in phases: one chunk q of every line (real types: two phases), for complex types one MFMA k
    // step h of it (four phases (h, q)).  The fragments of a phase are 2 A blocks and NJ B blocks, EPC batch entries each.
    constexpr int NPH = CX ? 4 : 2;
    constexpr int PH_MFMA = EPC * 2 * NJ;        // MFMAs per phase
    constexpr int NMF = NPH * PH_MFMA;           // ... per stage
    constexpr int ST_EVERY = NMF / (2 * KL);     // a store unit after every so many MFMAs
    static_assert(ST_EVERY >= 1 && ST_EVERY * 2 * KL == NMF, "store units divide the MFMAs of a stage");
    auto read_phase = [&](int buf, int ph, R (&fa_)[2][EPC], R (&fb_)[NJ][EPC]) __attribute__((always_inline)) {
        const unsigned char* sA = smem + buf * STAGE;
        const unsigned char* sB = sA + OPER;
        if constexpr (!CX) {
            const int q = ph;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const Chunk ca = *reinterpret_cast<const Chunk*>(sA + ((fa ^ (uint32_t)((16 * q) ^ (32 * i))) + (uint32_t)(i * 2048)));
                const Chunk cb = *reinterpret_cast<const Chunk*>(sB + ((fb ^ (uint32_t)((16 * q) ^ (32 * i))) + (uint32_t)(i * 2048)));
#pragma unroll
                for (int e = 0; e < EPC; ++e) {
                    fa_[i][e] = ca[e];
                    fb_[i][e] = cb[e];
                }
            }
        } else {
            const int h = ph >> 1, q = ph & 1;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const unsigned char* p = sA + ((fa ^ (uint32_t)((16 * q) ^ (32 * i))) + (uint32_t)(i * 2048 + h * 8192));
#pragma unroll
                for (int e = 0; e < EPC; ++e) fa_[i][e] = *reinterpret_cast<const R*>(p + e * 2 * (int)sizeof(R));
            }
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const unsigned char* p = sB + ((fb ^ (uint32_t)(16 * (q ^ j))) + (uint32_t)(j * 1024 + h * 8192));
#pragma unroll
                for (int e = 0; e < EPC; ++e) fb_[j][e] = *reinterpret_cast<const R*>(p + e * 2 * (int)sizeof(R));
            }
        }
    };
    // one stage: its MFMAs with, when STORE, the LDS stores of stage s_next (from register set x) spread between them;
    // the fragments of phase ph + 1 are read while phase ph is multiplied
    auto stage = [&](int buf, u4 (&x)[2 * KL]) __attribute__((always_inline)) {
        R FA[2][2][EPC], FB[2][NJ][EPC];
        read_phase(buf, 0, FA[0], FB[0]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ph = 0; ph < NPH; ++ph) {
            if (ph + 1 < NPH) read_phase(buf, ph + 1, FA[(ph + 1) & 1], FB[(ph + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const int q = CX ? (ph & 1) : ph;
#pragma unroll
            for (int e = 0; e < EPC; ++e)
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < NJ; ++j) {
                        R bv = FB[ph & 1][j][e];
                        if constexpr (CX) {   // -bi for (k part 1, column part 0)
                            if constexpr (sizeof(R) == 8) bv = __builtin_bit_cast(R, __builtin_bit_cast(uint64_t, bv) ^ ((uint64_t)bmask_hi << 32));
                            else bv = __builtin_bit_cast(R, __builtin_bit_cast(uint32_t, bv) ^ bmask_hi);
                        }
                        acc[q * EPC + e][i][j] = Mfma<R>::run(FA[ph & 1][i][e], bv, acc[q * EPC + e][i][j]);
                        const int m = ph * PH_MFMA + (e * 2 + i) * NJ + j;
                        if (m % ST_EVERY == ST_EVERY - 1) {
                            // the register that held the unit goes straight back to memory for the stage D further on: it is
                            // in flight for D whole iterations
                            store_unit(buf ^ 1, x, m / ST_EVERY, false);
                            load_unit(x, m / ST_EVERY, false);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
        }
    };

    // (the order of the loads is pinned: the wait counts of the loop assume that a register set's loads are the oldest
    // ones in flight when its turn to be stored comes)
#pragma unroll
    for (int u = 0; u < 2 * KL; ++u) load_unit(stg[0], u, true);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int d = 1; d < D; ++d) {
#pragma unroll
        for (int u = 0; u < 2 * KL; ++u) load_unit(stg[d], u, false);
        advance_loads();
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int u = 0; u < 2 * KL; ++u) {
        store_unit(0, stg[0], u, true);
        load_unit(stg[0], u, false);
        __builtin_amdgcn_sched_barrier(0);
    }
    advance_loads();
    __syncthreads();
    // Iteration t multiplies stage t out of LDS buffer t & 1; between its MFMAs stage t + 1 is stored, unit by unit, into
    // the other buffer from register set (t + 1) % D, and each register is loaded again at once, for stage t + 1 + D.
    // Every iteration is the same code: the loads past the last stage read valid memory again and their stores go
    // into a buffer that nobody reads any more.
    // (whole trips of D iterations first, the remaining ones after the loop: an exit from the middle of a trip would make
    // the compiler assume fewer loads in flight at the top of the loop and wait for the wrong ones)
    int s = 0;
    for (; s + D <= nstage; s += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            stage((s + d) & 1, stg[(d + 1) % D]);
            advance_loads();
            __syncthreads();
        }
    }
#pragma unroll
    for (int d = 0; d + 1 < D; ++d) {
        if (s + d < nstage) {
            stage((s + d) & 1, stg[(d + 1) % D]);
            advance_loads();
            __syncthreads();
        }
    }

    // ---- epilogue: C[batch, row, column], batch entries adjacent.  A lane holds, for its (row, column), the results of its
    // wave's batch entries only -- 16 or 32 bytes of that element's 128-byte line, the other waves hold the rest.  Stored
    // from the registers these pieces are 8192 scattered 16-byte writes per tile (measured: 134 MB of results took 107 us,
    // two thirds of the kernel).  Instead the tile goes through LDS, sixteen rows (512 lines, 64 KB) at a time: every wave
    // writes its chunks of the lines, then thread t stores chunk t % 8 of line (row p, column t / 8) in pass p, so that eight
    // lanes write one whole line.  A line's chunk c sits at position c ^ (line & 7): both sides are free of bank conflicts.
    const R ar = (R)g.alpha_re, ai = (R)g.alpha_im, br = (R)g.beta_re, bi = (R)g.beta_im;
    typedef typename RawVec<R, C_::RPC>::type OutV;
    typedef R OutU __attribute__((ext_vector_type(C_::RPC), aligned(sizeof(R))));
    // the storing thread: chunk c of column lr
    const bool st_ok = c < chunks_valid && lr < rowsB;
    R* Cst = reinterpret_cast<R*>(g.C) + (ob * g.sco + b0 + c * EPC + m0 * g.scm + (n0 + lr) * g.scn) * C_::EC;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        if (i > 0) __syncthreads();   // the stores of the first half have read their lines
        if constexpr (!CX) {
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int line = Mfma<R>::row(lane, r) * 32 + 16 * j + lrow;
                        OutV v;
#pragma unroll
                        for (int e = 0; e < EPC; ++e) v[e] = acc[q * EPC + e][i][j][r];
                        *reinterpret_cast<OutV*>(smem + line * 128 + (((2 * wave + q) ^ (line & 7)) << 4)) = v;
                    }
        } else {
            // even lanes hold the real parts, odd lanes the imaginary parts: each writes its half of the element
#pragma unroll
            for (int q = 0; q < 2; ++q)
#pragma unroll
                for (int j = 0; j < NJ; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int line = Mfma<R>::row(lane, r) * 32 + 8 * j + (lrow >> 1);
                        unsigned char* p = smem + line * 128 + (((2 * wave + q) ^ (line & 7)) << 4) + (lrow & 1) * (int)sizeof(R);
#pragma unroll
                        for (int e = 0; e < EPC; ++e) *reinterpret_cast<R*>(p + e * 2 * (int)sizeof(R)) = acc[q * EPC + e][i][j][r];
                    }
        }
        __syncthreads();
#pragma unroll
        for (int p = 0; p < 16; ++p) {
            const int line = p * 32 + lr;
            OutV v = *reinterpret_cast<const OutV*>(smem + line * 128 + ((c ^ (line & 7)) << 4));
            const int row = 16 * i + p;
            if (!st_ok || row >= rowsA) continue;
            R* dst = Cst + (int64_t)row * g.scm * C_::EC;
            OutV out;
            if constexpr (!CX) {
#pragma unroll
                for (int e = 0; e < EPC; ++e) out[e] = ar * v[e];
                if (g.use_beta) {
                    const OutV old = *reinterpret_cast<const OutU*>(dst);
#pragma unroll
                    for (int e = 0; e < EPC; ++e) out[e] += br * old[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < EPC; ++e) {
                    out[2 * e] = ar * v[2 * e] - ai * v[2 * e + 1];
                    out[2 * e + 1] = ar * v[2 * e + 1] + ai * v[2 * e];
                }
                if (g.use_beta) {
                    const OutV old = *reinterpret_cast<const OutU*>(dst);
#pragma unroll
                    for (int e = 0; e < EPC; ++e) {
                        out[2 * e] += br * old[2 * e] - bi * old[2 * e + 1];
                        out[2 * e + 1] += br * old[2 * e + 1] + bi * old[2 * e];
                    }
                }
            }
            *reinterpret_cast<OutU*>(dst) = out;
        }
    }
}

template <class R, bool CX, int D>
void launch_bfirst_t(const BfArgs& g, hipStream_t st) {
    typedef BfCfg<R, CX> C_;
    static bool once = [] {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_bfirst_kernel<R, CX, D>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)C_::LDS_BYTES);
        return true;
    }();
    (void)once;
    const uint64_t blocks = (uint64_t)g.tiles_m * (uint64_t)g.tiles_n * (uint64_t)g.groups * (uint64_t)g.nbo;
    TFH_LAUNCH_TIMED((gemm_bfirst_kernel<R, CX, D>), dim3((uint32_t)blocks), dim3(256), (size_t)C_::LDS_BYTES, st, g);
}

}  // namespace gemm

namespace {
void sort_by_c(std::vector<Axis>& ax) {
    std::stable_sort(ax.begin(), ax.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[2]) > std::llabs(y.s[2]); });
}
}  // namespace

// Returns false when the shape is not one this kernel takes; true when it launched (status holds the outcome).
int32_t launch_batch_first(int dtype, const gemm::BfArgs& g, void* stream) {
    using namespace gemm;
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_CONTRACT, stream);
    switch (dtype) {
        case TFH_F32: launch_bfirst_t<float, false, 2>(g, st); break;
        case TFH_F64: launch_bfirst_t<double, false, 2>(g, st); break;
        case TFH_C64: launch_bfirst_t<float, true, 2>(g, st); break;
        default: launch_bfirst_t<double, true, 2>(g, st); break;
    }
    prof_end(prof, stream);
    return hip_check(hipGetLastError(), "batch-first contraction kernel");
}

bool try_batch_first(int dtype, const void* a, const void* b, void* c, const ContractAxes& ax0, Scalar alpha, Scalar beta,
                     void* stream, bool conj_a, bool conj_b, int32_t& status, gemm::BfArgs* routed) {
    using namespace gemm;
    if (ax0.batch.empty() || ax0.M.empty() || ax0.N.empty() || ax0.K.empty()) return false;
    const int64_t eb = (int64_t)dtype_size(dtype);
    const int64_t epc = 16 / eb, nbk = 8 * epc;
    ContractAxes ax = ax0;
    sort_by_c(ax.batch);
    sort_by_c(ax.M);
    sort_by_c(ax.N);
    std::stable_sort(ax.K.begin(), ax.K.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[0]) > std::llabs(y.s[0]); });
    fuse_axes(ax.batch, 3);
    fuse_axes(ax.M, 3);
    fuse_axes(ax.N, 3);
    fuse_axes(ax.K, 3);
    if (ax.batch.empty() || ax.batch.size() > 2 || ax.M.size() != 1 || ax.N.size() != 1 || ax.K.size() != 1) return false;
    const Axis& bi = ax.batch.back();
    if (bi.s[0] != 1 || bi.s[1] != 1 || bi.s[2] != 1) return false;
    if (bi.n % epc != 0 || bi.n < 2 * nbk) return false;
    const Axis &m = ax.M[0], &n = ax.N[0], &k = ax.K[0];
    if (m.n < 2 || n.n < 2) return false;
    if (m.s[0] < 0 || m.s[2] <= 0 || n.s[1] < 0 || n.s[2] <= 0 || k.s[0] < 0 || k.s[1] < 0) return false;
    // per-thread 32-bit byte offsets span one tile's rows
    if (32 * m.s[0] * eb + 256 >= ((int64_t)1 << 31) || 32 * n.s[1] * eb + 256 >= ((int64_t)1 << 31)) return false;
    BfArgs g;
    std::memset(&g, 0, sizeof g);
    g.A = a; g.B = b; g.C = c;
    g.nb = bi.n;
    g.nbo = 1;
    if (ax.batch.size() == 2) {
        g.nbo = ax.batch[0].n;
        g.sao = ax.batch[0].s[0]; g.sbo = ax.batch[0].s[1]; g.sco = ax.batch[0].s[2];
    }
    g.M = m.n; g.N = n.n; g.K = k.n;
    g.sam = m.s[0]; g.scm = m.s[2];
    g.sbn = n.s[1]; g.scn = n.s[2];
    g.sak = k.s[0]; g.sbk = k.s[1];
    g.tiles_m = (int32_t)((g.M + 31) / 32);
    g.tiles_n = (int32_t)((g.N + 31) / 32);
    g.groups = (int32_t)((g.nb + nbk - 1) / nbk);
    const uint64_t blocks = (uint64_t)g.tiles_m * (uint64_t)g.tiles_n * (uint64_t)g.groups * (uint64_t)g.nbo;
    if (blocks == 0 || blocks > 0x7fffffffull || g.M > ((int64_t)1 << 30) || g.N > ((int64_t)1 << 30)) return false;
    g.conj_a = conj_a; g.conj_b = conj_b;
    g.use_beta = !beta.is_zero();
    g.alpha_re = alpha.re; g.alpha_im = alpha.im; g.beta_re = beta.re; g.beta_im = beta.im;
    if (routed) *routed = g;
    status = launch_batch_first(dtype, g, stream);
    return true;
}

}  // namespace tfh
