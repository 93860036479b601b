// k_gemm_skinny.hip -- contraction with a small left operand: C[m, n] = alpha * sum_k A[m, k] * B[n, k] + beta * C
// with at most 32 rows m, at most 32 16-byte chunks of k (64 real k in double, 128 in single precision), and a long n
// (the "apply a small operator to every fibre of a large tensor" step of a tensor-network contraction,
// PrimDescriptor::Contract, tenferro-prims/src/lib.rs:227-239).  All four dtypes.
//
// Such a product is bound by HBM (B is read once, C written once, a few flops per byte), and a tiled GEMM kernel
// spends it in per-tile latency: with so little k there is no main loop to hide the loads and the stores behind.
// Here A lives in registers, already laid out as MFMA operands, for the whole kernel, and every wave streams B on
// its own: a work unit is 16 consecutive n; the wave loads the unit's rows of B (k contiguous) with 16-byte
// accesses into registers, parks them in its private LDS region, has the next unit's loads in flight while the
// MFMAs of the current one run, and writes the unit's columns of C from the accumulators one unit later, among the
// MFMAs of the next unit.  Waves never wait for each other (no block barrier).
//
// v_mfma_f64_16x16x4_f64: lane l = 16 g + j feeds A'[row j][k' = 4 step + g] and B'[k' = 4 step + g][col j] and
// receives C'[row g + 4 r][col j] in accumulator register r (v_mfma_f32_16x16x4_f32: row 4 g + r).  One 16-byte chunk
// of B serves two steps in double precision (four in single: twice the components per chunk, otherwise alike):
//   complex128: chunk c of row n is the element B[n][k = c] = (br, bi).  Real form of the product: A'[m][2k + q] =
//     (re, im)[q] of A[m][k]; B'[2k][2n] = br, B'[2k+1][2n] = -bi, B'[2k][2n+1] = bi, B'[2k+1][2n+1] = br; C'[m][2n + p]
//     is the interleaved complex C.  Column j is (n = j / 2, p = j % 2): the lane turns its chunk into the operands
//     (p ? bi : br) for q = 0 and (p ? br : -bi) for q = 1.  Two column blocks (16 n) per unit.
//   f64: chunk c of row n holds B[n][2c], B[n][2c+1], the operands of q = 0, 1.  Column j is n.  One column block.
// Pair i of steps (2i, 2i+1) uses chunk 4i + g in lane group g: a permutation of k shared by A' and B', harmless
// under the sum.  HBM-bound: algorithmic bytes = sizeof(B) + sizeof(C) (+ C again when beta != 0).
//
// B may also be contiguous along n instead of k (the operator acts on a leg that is not the tensor's last): the unit
// is then parked as [k][16 n] and an MFMA operand is one element of the park (see NFAST below).
//
// C may be contiguous along n (each lane stores its accumulators: 128-byte segments per row of C) or along m (the
// other orientation of the same product, C[n][m]): then the unit's 16 x M results are transposed through an LDS tile
// of the wave's own and leave as 16-byte stores along m.
#include <hip/hip_runtime.h>

#include "gemm_skinny.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

using namespace gemm;

// A 16-byte chunk: two doubles or four floats
template <class R> struct Chunk;
template <> struct Chunk<double> { typedef double type __attribute__((ext_vector_type(2))); };
template <> struct Chunk<float> { typedef float type __attribute__((ext_vector_type(4))); };
// N components read from LDS at once
template <class R, int N> struct Comps { typedef R type __attribute__((ext_vector_type(N))); };
template <class R> struct Comps<R, 1> { typedef R type; };
template <int Q, class V> __device__ __forceinline__ auto comp_of(const V& v, int q) {
    if constexpr (Q == 1) return v;
    else return v[q];
}

// Sizes of one instantiation: R the component type, KCM 16-byte chunks per row of B at most, MBM blocks of 16 rows of A
// at most.  The general kernel (32 chunks, 2 blocks) keeps 64 VGPRs of A (doubles) and 32 of staging and runs two waves
// per SIMD; an operator of at most 16 rows and 8 chunks needs a tenth of that, and twice as many waves hide twice the
// latency of its short units.
template <class R, int KCM, int MBM>
struct SkinnyCfg {
    static constexpr int Q = 16 / (int)sizeof(R);             // components per chunk
    static constexpr int MAX_KC = KCM;
    static constexpr int PITCH = MAX_KC * 16 + 64;            // bytes per LDS row: rows 0..3 start 16 banks apart
    static constexpr int WAVE_LDS = SKINNY_UNIT * PITCH;      // each wave parks one unit
    static constexpr int LOADS = SKINNY_UNIT * MAX_KC / 64;   // 16-byte loads per lane and unit at most
    static constexpr int PAIRS = MAX_KC / 4;
    static constexpr int OLOADS = SKINNY_UNIT * (32 * MBM / Q) / 64;   // 16-byte pieces of the result tile per lane at most (complex)
    static constexpr int OUT_PITCH = 2 * 16 * MBM + Q;        // components per row of the transposed result tile (+16 bytes against bank conflicts)
    static constexpr int TILE_LDS = SKINNY_UNIT * OUT_PITCH * (int)sizeof(R);   // the transposed result tile of a wave: a region of its own
    static constexpr int BLOCKS_PER_CU = KCM <= 8 && MBM == 1 ? 4 : 2;
    // B contiguous along n instead of k: the unit is parked as [k][16 n], at most MAX_KC rows of k
    template <bool CX> struct Nfast {
        static constexpr int ELEM = (CX ? 2 : 1) * (int)sizeof(R);      // bytes per element
        static constexpr int ROW_CHUNKS = SKINNY_UNIT * ELEM / 16;      // 16-byte chunks per k row
        // bytes per k row: the lane groups g = 0..3 (four consecutive k) start on different banks
        static constexpr int KPITCH = SKINNY_UNIT * ELEM + (ELEM == 4 ? 16 : 64);
        static constexpr int WAVE_LDS = MAX_KC * KPITCH;
        static constexpr int LOADS = (MAX_KC * ROW_CHUNKS + 63) / 64;
    };
    static_assert(KCM % 4 == 0 && KCM <= SKINNY_MAX_CHUNKS && MBM * 16 <= SKINNY_MAX_M, "");
};

// Orders the LDS accesses of one wave: lanes read what other lanes of the same wave wrote.  The LDS executes a wave's
// instructions in order, so only the compiler has to be kept from moving accesses across this point.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// RAGGED: the innermost run of n holds no whole number of units (its own instantiation: the full-unit kernel carries
// none of the per-unit predicates).  OUT_ROWS: C is contiguous along m (s.out_rows).  NFAST (either output): B is
// contiguous along n, not along k -- the operator acts on a leg that is not the tensor's last: a unit is then K
// segments of 16 consecutive n, parked as [k][n]; an MFMA operand is one element of it (lane group g takes k = 4t + g
// in step t), where the k-contiguous form reads a 16-byte chunk of one row for several steps.
//
// vmcnt counts loads and stores in one queue, in order, and the compiler waits for a register that was loaded in the
// iteration before with vmcnt(0): whatever is stored shortly before that wait is waited for as well, acknowledgement
// included.  With C contiguous along n a unit's results therefore stay in registers for one more iteration and leave
// in the middle of the next unit's MFMAs: by the time the next wait comes, they have had half an iteration to drain.
template <class R, bool CX, bool RAGGED, bool OUT_ROWS, int KCM, int MBM, bool NFAST = false>
__global__ void __launch_bounds__(THREADS, (SkinnyCfg<R, KCM, MBM>::BLOCKS_PER_CU)) gemm_skinny_kernel(SkinnyArgs s) {
    typedef SkinnyCfg<R, KCM, MBM> Cfg;
    typedef typename Cfg::template Nfast<CX> Nf;
    typedef typename Chunk<R>::type chunk_t;
    typedef typename Mfma<R>::acc_t acc_t;
    constexpr int PITCH = Cfg::PITCH, WAVE_LDS = NFAST ? Nf::WAVE_LDS : Cfg::WAVE_LDS, LOADS = NFAST ? Nf::LOADS : Cfg::LOADS;
    constexpr int PAIRS = Cfg::PAIRS, Q = Cfg::Q, KPITCH = Nf::KPITCH;
    constexpr int QB = NFAST ? (CX ? 2 : 1) : Q;   // components per LDS read = MFMA steps per read
    constexpr int OUT_PITCH = Cfg::OUT_PITCH, TILE_LDS = Cfg::TILE_LDS, OLOADS = Cfg::OLOADS;
    constexpr int NBLK = CX ? 2 : 1;   // column blocks (16 real columns each) per unit
    constexpr int NC = CX ? 2 : 1;     // components per element
    constexpr int EB = (int)sizeof(R);
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    unsigned char* lds = smem + wave * (WAVE_LDS + (OUT_ROWS ? TILE_LDS : 0));
    unsigned char* tile_lds = lds + WAVE_LDS;   // OUT_ROWS only
    const int g = lane >> 4, j = lane & 15, p = j & 1;
    const int kc = s.kc, npair = ((NFAST ? s.K : kc) + 3) >> 2, nmb = MBM > 1 && s.M > 16 ? 2 : 1;

    // ---- A as MFMA operands: a[mb][i][q] = A'[j + 16 mb][QB (4i + g) + q], zero outside the matrix.  A' is A itself for
    // real elements and its real form for complex ones: A'[m][2k + part] = (re, im)[part] of A[m][k].
    R a[MBM][PAIRS][QB];
    {
        // (indices past the matrix are redirected to its last row and last k and the values dropped afterwards: without a
        // branch per element all of a lane's loads are in flight together -- with 32 units per wave at a million columns
        // this prologue is not small; a complex element is one load of both parts)
        const R* Ad = reinterpret_cast<const R*>(s.A);
        typedef R Pair __attribute__((ext_vector_type(2), aligned(sizeof(R))));
#pragma unroll
        for (int mb = 0; mb < MBM; ++mb)
#pragma unroll
            for (int i = 0; i < PAIRS; ++i) {
                const int m = j + 16 * mb, c = 4 * i + g;
                const int64_t mo = off_of(s.am, m < s.M ? m : s.M - 1);
                if constexpr (CX) {
#pragma unroll
                    for (int e = 0; e < QB / 2; ++e) {
                        const int k = (QB / 2) * c + e;
                        const bool ok = m < s.M && k < s.K;
                        const Pair v = *reinterpret_cast<const Pair*>(Ad + 2 * (mo + off_of(s.ak, k < s.K ? k : s.K - 1)));
                        a[mb][i][2 * e] = ok ? v[0] : R(0);
                        a[mb][i][2 * e + 1] = ok ? (s.conj_a ? -v[1] : v[1]) : R(0);
                    }
                } else {
#pragma unroll
                    for (int q = 0; q < QB; ++q) {
                        const int k = QB * c + q;
                        const R x = Ad[mo + off_of(s.ak, k < s.K ? k : s.K - 1)];
                        a[mb][i][q] = (m < s.M && k < s.K) ? x : R(0);
                    }
                }
            }
    }

    // ---- this lane's share of a unit of B: chunk id = lane + 64 u -> (row, chunk of the row)
    int32_t goff[LOADS], loff[LOADS];
    uint32_t have = 0, lrows = 0;   // lrows: four bits per load, the n of the unit it belongs to
    static_assert(LOADS <= 8 && OLOADS <= 8 && SKINNY_UNIT <= 16, "row numbers are packed four bits per load or store");
#pragma unroll
    for (int u = 0; u < LOADS; ++u) {
        const int id = lane + 64 * u;
        if constexpr (NFAST) {
            // chunk id -> (k, chunk of the 16 n); the first n of the chunk goes into lrows
            const bool ok = id < s.K * Nf::ROW_CHUNKS;
            const int krow = id / Nf::ROW_CHUNKS, ch = id % Nf::ROW_CHUNKS;
            have |= (ok ? 1u : 0u) << u;
            lrows |= (ok ? (uint32_t)(ch * (16 / Nf::ELEM)) : 0u) << (4 * u);
            goff[u] = ok ? (int32_t)(off_of(s.bk, krow) * Nf::ELEM) + ch * 16 : 0;
            loff[u] = ok ? krow * KPITCH + ch * 16 : 0;
        } else {
        const bool ok = id < SKINNY_UNIT * kc;
        const int row = id / kc, col = id - row * kc;   // (n, chunk of its k)
        have |= (ok ? 1u : 0u) << u;
        lrows |= (ok ? (uint32_t)row : 0u) << (4 * u);
        {
            goff[u] = ok ? row * s.b_in * (EB * NC) + col * 16 : 0;
            loff[u] = ok ? row * PITCH + col * 16 : 0;
        }
        }
    }
    // ---- where this lane reads its operands and writes its results
    int32_t roff[NBLK], ccol[NBLK] = {}, crow[MBM][4] = {};
#pragma unroll
    for (int nb = 0; nb < NBLK; ++nb) {
        const int nloc = CX ? 8 * nb + (j >> 1) : j;
        roff[nb] = NFAST ? g * KPITCH + nloc * Nf::ELEM : nloc * PITCH + g * 16;
        if constexpr (!OUT_ROWS) ccol[nb] = nloc * s.c_in * NC + (CX ? p : 0);
    }
    if constexpr (!OUT_ROWS) {
#pragma unroll
        for (int mb = 0; mb < MBM; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = Mfma<R>::row(lane, r) + 16 * mb;
                crow[mb][r] = m < s.M ? (int32_t)(off_of(s.cm, m) * NC) : 0;
            }
    }
    const R ar = (R)s.alpha_re, ai = (R)s.alpha_im, br = (R)s.beta_re, bi = (R)s.beta_im;
    // C contiguous along m: 16-byte piece id = lane + 64 u of the unit's result tile -> (n of the unit, piece of its row)
    int32_t ogoff[OLOADS] = {}, oloff[OLOADS] = {};
    uint32_t ohave = 0, orows = 0;
    if constexpr (OUT_ROWS) {
        const int cpr = s.M * NC / Q;   // 16-byte pieces per row of C
#pragma unroll
        for (int u = 0; u < OLOADS; ++u) {
            const int id = lane + 64 * u, row = id / cpr, col = id - row * cpr;
            const bool ok = id < SKINNY_UNIT * cpr;
            ohave |= (ok ? 1u : 0u) << u;
            orows |= (ok ? (uint32_t)row : 0u) << (4 * u);
            ogoff[u] = ok ? (row * s.c_in * NC + col * Q) * EB : 0;
            oloff[u] = ok ? (row * OUT_PITCH + col * Q) * EB : 0;
        }
    }

    const int64_t nwaves = (int64_t)gridDim.x * (THREADS / 64);
    int64_t unit = (int64_t)blockIdx.x * (THREADS / 64) + wave;
    chunk_t stage[LOADS];
    // The innermost run of n need not hold a whole number of units: the last unit of each run then has s.tail valid n.
    // Rows past them are neither loaded (what is parked for them is whatever the registers held: their columns of the
    // product are independent of the others and never stored) nor written.
    auto valid_of = [&](int64_t un) -> int {
        if constexpr (!RAGGED) return SKINNY_UNIT;
        return (int)(un % s.upr) == s.upr - 1 ? s.tail : SKINNY_UNIT;
    };
    auto issue = [&](int64_t un) {
        const unsigned char* Bu = reinterpret_cast<const unsigned char*>(s.B) + off_of(s.bu, un) * (EB * NC);
        const int valid = valid_of(un);
#pragma unroll
        for (int u = 0; u < LOADS; ++u)
            if (((have >> u) & 1u) && (int)((lrows >> (4 * u)) & 15u) < valid)
                stage[u] = __builtin_nontemporal_load(reinterpret_cast<const chunk_t*>(Bu + goff[u]));
    };
    // C contiguous along n: lane (g, j) holds the rows Mfma<R>::row(lane, r) (+16), column j of each column block
    auto store_direct = [&](const acc_t (&res)[MBM][NBLK], R* Cu, int valid) {
#pragma unroll
        for (int mb = 0; mb < MBM; ++mb) {
            if (mb < nmb) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const bool row_ok = Mfma<R>::row(lane, r) + 16 * mb < s.M;
#pragma unroll
                    for (int nb = 0; nb < NBLK; ++nb) {
                        const bool ok = row_ok && (CX ? 8 * nb + (j >> 1) : j) < valid;
                        R* dst = Cu + crow[mb][r] + ccol[nb];
                        R v = res[mb][nb][r];
                        if (!s.plain) {
                            if constexpr (CX) {
                                // even lanes hold re, odd lanes im of one element: exchange with the neighbour
                                const R other = __shfl_xor(v, 1);
                                const R re_v = p ? other : v, im_v = p ? v : other;
                                v = p ? (ar * im_v + ai * re_v) : (ar * re_v - ai * im_v);
                                if (s.use_beta) {
                                    const R old = ok ? *dst : R(0);
                                    const R old_other = __shfl_xor(old, 1);
                                    const R re_o = p ? old_other : old, im_o = p ? old : old_other;
                                    v += p ? (br * im_o + bi * re_o) : (br * re_o - bi * im_o);
                                }
                            } else {
                                v *= ar;
                                if (s.use_beta && ok) v += br * *dst;
                            }
                        }
                        if (ok) __builtin_nontemporal_store(v, dst);
                    }
                }
            }
        }
    };
    // C contiguous along m: the tile of the unit before leaves as 16-byte pieces of whole rows
    auto store_rows = [&](R* Cu, int valid) {
#pragma unroll
        for (int u = 0; u < OLOADS; ++u)
            if (((ohave >> u) & 1u) && (int)((orows >> (4 * u)) & 15u) < valid) {
                chunk_t v = *reinterpret_cast<const chunk_t*>(tile_lds + oloff[u]);
                chunk_t* dst = reinterpret_cast<chunk_t*>(reinterpret_cast<unsigned char*>(Cu) + ogoff[u]);
                if (!s.plain) {
                    chunk_t o;
                    if constexpr (CX) {
#pragma unroll
                        for (int e = 0; e < Q; e += 2) {
                            o[e] = ar * v[e] - ai * v[e + 1];
                            o[e + 1] = ar * v[e + 1] + ai * v[e];
                        }
                        if (s.use_beta) {
                            const chunk_t old = *dst;
#pragma unroll
                            for (int e = 0; e < Q; e += 2) {
                                o[e] += br * old[e] - bi * old[e + 1];
                                o[e + 1] += br * old[e + 1] + bi * old[e];
                            }
                        }
                    } else {
                        o = v * ar;
                        if (s.use_beta) o += *dst * br;
                    }
                    v = o;
                }
                __builtin_nontemporal_store(v, dst);
            }
    };
    acc_t held[MBM][NBLK];     // !OUT_ROWS: the results of the unit before, not yet stored (OUT_ROWS: they wait in the tile)
    R* held_c = nullptr;
    int held_valid = 0;
#pragma unroll
    for (int u = 0; u < LOADS; ++u)
#pragma unroll
        for (int e = 0; e < Q; ++e) stage[u][e] = 0;
    if (unit < s.units) issue(unit);
    while (unit < s.units) {
        const int valid = valid_of(unit);
#pragma unroll
        for (int u = 0; u < LOADS; ++u)
            if ((have >> u) & 1u) *reinterpret_cast<chunk_t*>(lds + loff[u]) = stage[u];
        const int64_t next = unit + nwaves;
        // (a table lookup here finds nothing else in flight: behind the loads of the next unit it would wait for them)
        R* Cu = reinterpret_cast<R*>(s.C) + off_of(s.cu, unit) * NC;
        if (next < s.units) issue(next);
        wave_sync();

        acc_t acc[MBM][NBLK];
#pragma unroll
        for (int mb = 0; mb < MBM; ++mb)
#pragma unroll
            for (int nb = 0; nb < NBLK; ++nb) acc[mb][nb] = acc_t{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < PAIRS; ++i) {
            if (i < npair) {
                const bool kok = 4 * i + g < (NFAST ? s.K : kc);
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) {
                    typedef typename Comps<R, QB>::type read_t;
                    const read_t ch = *reinterpret_cast<const read_t*>(lds + roff[nb] + i * (NFAST ? 4 * KPITCH : 64));
                    // the chunk as operands B'[Q c + q][column j]: the components themselves for real elements; for a
                    // complex element (br, bi) the even column of its pair takes (br, -bi), the odd one (bi, br)
                    R b[QB];
#pragma unroll
                    for (int q = 0; q < QB; ++q) {
                        if constexpr (CX) {
                            const R re = ch[q & ~1], im = s.conj_b ? -ch[q | 1] : ch[q | 1];
                            b[q] = (q & 1) ? (p ? re : -im) : (p ? im : re);
                        } else {
                            b[q] = comp_of<QB>(ch, q);
                        }
                        b[q] = kok ? b[q] : R(0);   // a row of B may be shorter than the LDS row: never multiply what was not loaded
                    }
#pragma unroll
                    for (int q = 0; q < QB; ++q) acc[0][nb] = Mfma<R>::run(a[0][i][q], b[q], acc[0][nb]);
                    if constexpr (MBM > 1)
                        if (nmb > 1) {
#pragma unroll
                            for (int q = 0; q < QB; ++q) acc[1][nb] = Mfma<R>::run(a[1][i][q], b[q], acc[1][nb]);
                        }
                }
            }
            if (i == 0 && held_c) {
                if constexpr (OUT_ROWS) store_rows(held_c, held_valid);
                else store_direct(held, held_c, held_valid);
            }
        }
        wave_sync();   // the next unit is parked over these rows, and its results are written over the tile

        if constexpr (OUT_ROWS) {
            // tile[n of the unit][m][part] in LDS; whole rows leave during the next unit's MFMAs (store_rows)
            R* tile = reinterpret_cast<R*>(tile_lds);
#pragma unroll
            for (int mb = 0; mb < MBM; ++mb)
                if (mb < nmb) {
#pragma unroll
                    for (int r = 0; r < 4; ++r)
#pragma unroll
                        for (int nb = 0; nb < NBLK; ++nb) {
                            const int m = Mfma<R>::row(lane, r) + 16 * mb, nloc = CX ? 8 * nb + (j >> 1) : j;
                            tile[nloc * OUT_PITCH + m * NC + (CX ? p : 0)] = acc[mb][nb][r];
                        }
                }
            held_c = Cu;
            held_valid = valid;
        }
        if constexpr (!OUT_ROWS) {
#pragma unroll
            for (int mb = 0; mb < MBM; ++mb)
#pragma unroll
                for (int nb = 0; nb < NBLK; ++nb) held[mb][nb] = acc[mb][nb];
            held_c = Cu;
            held_valid = valid;
        }
        unit = next;
    }
    if (held_c) {
        if constexpr (OUT_ROWS) {
            wave_sync();
            store_rows(held_c, held_valid);
        } else {
            store_direct(held, held_c, held_valid);
        }
    }
}

template <class R, bool CX, bool RAGGED, bool OUT_ROWS, int KCM, int MBM, bool NFAST = false>
void launch_variant(const gemm::SkinnyArgs& s, hipStream_t st) {
    typedef SkinnyCfg<R, KCM, MBM> Cfg;
    constexpr int lds = (THREADS / 64) * ((NFAST ? Cfg::template Nfast<CX>::WAVE_LDS : Cfg::WAVE_LDS) + (OUT_ROWS ? Cfg::TILE_LDS : 0));
    static bool once = [] {   // (more than 64 KB of dynamic LDS has to be asked for once per kernel)
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_skinny_kernel<R, CX, RAGGED, OUT_ROWS, KCM, MBM, NFAST>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        return true;
    }();
    (void)once;
    const int64_t blocks_wanted = (s.units + THREADS / 64 - 1) / (THREADS / 64);
    const dim3 grid((uint32_t)std::min<int64_t>(blocks_wanted, 256 * Cfg::BLOCKS_PER_CU)), block(THREADS);
    TFH_LAUNCH_TIMED((gemm_skinny_kernel<R, CX, RAGGED, OUT_ROWS, KCM, MBM, NFAST>), grid, block, (size_t)lds, st, s);
}

template <class R, bool CX, bool RAGGED, bool OUT_ROWS>
void launch_sized(const gemm::SkinnyArgs& s, hipStream_t st) {
    // (twice the waves pay where a unit is short: measured faster up to 8 complex or 16 real rows, even beyond)
    if (s.kc <= 8 && s.M <= (CX ? 8 : 16)) launch_variant<R, CX, RAGGED, OUT_ROWS, 8, 1>(s, st);
    else launch_variant<R, CX, RAGGED, OUT_ROWS, SKINNY_MAX_CHUNKS, SKINNY_MAX_M / 16>(s, st);
}

template <class R, bool CX>
void launch_typed(const gemm::SkinnyArgs& s, hipStream_t st) {
    const bool ragged = s.tail != 0, rows = s.out_rows != 0;
    if (ragged) {
        if (rows) launch_sized<R, CX, true, true>(s, st);
        else launch_sized<R, CX, true, false>(s, st);
    } else {
        if (rows) launch_sized<R, CX, false, true>(s, st);
        else launch_sized<R, CX, false, false>(s, st);
    }
}

template <class R, bool CX, bool RAGGED, bool OUT_ROWS>
void launch_nfast_sized(const gemm::SkinnyArgs& s, hipStream_t st) {
    if (s.K <= 8 && s.M <= (CX ? 8 : 16)) launch_variant<R, CX, RAGGED, OUT_ROWS, 8, 1, true>(s, st);
    else launch_variant<R, CX, RAGGED, OUT_ROWS, SKINNY_MAX_CHUNKS, SKINNY_MAX_M / 16, true>(s, st);
}

template <class R, bool CX>
void launch_nfast(const gemm::SkinnyArgs& s, hipStream_t st) {
    const bool ragged = s.tail != 0, rows = s.out_rows != 0;
    if (ragged) {
        if (rows) launch_nfast_sized<R, CX, true, true>(s, st);
        else launch_nfast_sized<R, CX, true, false>(s, st);
    } else {
        if (rows) launch_nfast_sized<R, CX, false, true>(s, st);
        else launch_nfast_sized<R, CX, false, false>(s, st);
    }
}

void launch_gemm_skinny_impl(int dtype, const gemm::SkinnyArgs& s, hipStream_t st) {
    if (s.nfast) {   // at most SKINNY_MAX_CHUNKS k (the host's conditions)
        switch (dtype) {
            case TFH_F32: launch_nfast<float, false>(s, st); break;
            case TFH_F64: launch_nfast<double, false>(s, st); break;
            case TFH_C64: launch_nfast<float, true>(s, st); break;
            default: launch_nfast<double, true>(s, st); break;
        }
        return;
    }
    switch (dtype) {
        case TFH_F32: launch_typed<float, false>(s, st); break;
        case TFH_F64: launch_typed<double, false>(s, st); break;
        case TFH_C64: launch_typed<float, true>(s, st); break;
        default: launch_typed<double, true>(s, st); break;
    }
}

}  // namespace

void launch_gemm_skinny(int dtype, const gemm::SkinnyArgs& s, hipStream_t st) { launch_gemm_skinny_impl(dtype, s, st); }

}  // namespace tfh
