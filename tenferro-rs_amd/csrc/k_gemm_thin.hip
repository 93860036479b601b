// k_gemm_thin.hip -- contraction of a long operand with a small one whose rows or k are too many for the register-
// resident streaming kernel (k_gemm_skinny.hip): C[n, m] = alpha * sum_k L[n, k] * S[m, k] + beta * C with up to 32 real
// rows of S (16 complex), S no larger than 64 KB, and a long n whose rows of L are contiguous in k
// (PrimDescriptor::Contract, tenferro-prims/src/lib.rs:227-239: 32 x 128 or 32 x 256 against a million rows, 16 x 512).
// All four dtypes.
//
// Such a product moves a few flops per byte: it is bound by HBM (and, in double precision from 32 rows on, close to
// the matrix cores as well), and tiles of a GEMM kernel spend it in per-tile latency, half of each tile empty.  Here S
// is staged once per block in LDS, already laid out as MFMA operands (and, for complex types, already expanded to the
// real matrix [[re, -im], [im, re]] with the conjugations folded in, so that the long operand is used as it lies in
// memory, as rows of 2 K reals), and every wave streams L on its own: a work unit is 16 consecutive n; a lane loads
// 16-byte chunks of its row straight into MFMA operand position (lane l = 16 g + j takes chunk 4 i + g of row j in
// step i: a permutation of k that S's layout shares), eight chunks per lane in flight behind the eight being
// multiplied, across unit boundaries.  No block barrier after the staging.  A unit's 16 x M results leave through a
// tile of the wave's own in LDS, so that they are stored along whichever index C is contiguous in, with alpha and
// beta applied where a lane holds whole elements.  HBM-bound: algorithmic bytes = sizeof(L) + sizeof(C).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

#include "gemm_common.hpp"
#include "internal.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

using namespace gemm;

constexpr int THIN_THREADS = 512, THIN_WAVES = THIN_THREADS / 64;
constexpr int THIN_UNIT = 16;          // consecutive n per work unit
constexpr int THIN_GROUP = 8;          // chunk steps (one 16-byte load per lane each) per register set
constexpr int THIN_S_BYTES = 64 * 1024;

struct ThinArgs {
    const void* S;
    const void* L;
    void* C;
    int32_t ms, K;            // rows of S and contracted extent, in elements
    int32_t mr, kr;           // the same in reals
    int32_t steps;            // chunk steps per row: ceil(16-byte chunks per row / 4)
    int32_t groups;           // ceil(steps / THIN_GROUP)
    int32_t cx, conj_s, conj_l, use_beta;
    int32_t m_fast;           // C is contiguous along m, not along n
    int64_t nl, units;        // rows of L; work units
    int64_t ss_m, ss_k;       // element strides of S
    int64_t ls_n;             // element stride between rows of L (k has stride 1)
    int64_t cs_m, cs_n;       // element strides of C
    double alpha_re, alpha_im, beta_re, beta_im;
};

template <class R> struct ThinChunk;
template <> struct ThinChunk<double> { typedef double type __attribute__((ext_vector_type(2))); };
template <> struct ThinChunk<float> { typedef float type __attribute__((ext_vector_type(4))); };

__device__ __forceinline__ void thin_wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// MB: blocks of 16 real rows of S.
template <class R, int MB>
__global__ void __launch_bounds__(THIN_THREADS, 2) gemm_thin_kernel(ThinArgs a) {
    constexpr int Q = 16 / (int)sizeof(R);   // reals per chunk = MFMA steps per chunk step
    typedef typename ThinChunk<R>::type Chunk;
    typedef typename Mfma<R>::acc_t Acc;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, j = lane & 15;
    const int steps_p = a.groups * THIN_GROUP;               // chunk steps, padded to whole register sets
    Chunk* As = reinterpret_cast<Chunk*>(smem_raw);          // [MB][steps_p][64 lanes]
    constexpr int TP = MB * 16 + 1;                          // pitch of the result tile in reals (odd: no bank conflicts)
    R* tile = reinterpret_cast<R*>(smem_raw + (size_t)MB * steps_p * 64 * 16) + (size_t)wave * THIN_UNIT * TP;
    // ---- stage S: entry (mb, i, lane) holds S'[16 mb + j][Q (4 i + g) + q], q < Q
    {
        const R* S = reinterpret_cast<const R*>(a.S);
        const int nc = a.cx ? 2 : 1;
        const double sgn_s = a.conj_s ? -1.0 : 1.0, sgn_l = a.conj_l ? -1.0 : 1.0;
        for (int e = tid; e < MB * steps_p * 64; e += THIN_THREADS) {
            const int l = e & 63, i = (e >> 6) % steps_p, mb = (e >> 6) / steps_p;
            const int row = 16 * mb + (l & 15);
            Chunk v;
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int kk = Q * (4 * i + (l >> 4)) + q;
                R x = R(0);
                if (row < a.mr && kk < a.kr) {
                    if (!a.cx) {
                        x = S[(int64_t)row * a.ss_m + (int64_t)kk * a.ss_k];
                    } else {
                        const int m = row >> 1, p = row & 1, k = kk >> 1, t = kk & 1;
                        const R* el = S + ((int64_t)m * a.ss_m + (int64_t)k * a.ss_k) * nc;
                        const double sr = el[0], si = sgn_s * (double)el[1];
                        // Re = lr sr - (sgn_l li) si,  Im = lr si + (sgn_l li) sr, against the row (lr, li) as it lies in memory
                        x = (R)(p == 0 ? (t == 0 ? sr : -sgn_l * si) : (t == 0 ? si : sgn_l * sr));
                    }
                }
                v[q] = x;
            }
            As[e] = v;
        }
    }
    __syncthreads();
    // ---- stream L
    const R* L = reinterpret_cast<const R*>(a.L);
    const int nc = a.cx ? 2 : 1;
    const int64_t wave_id = (int64_t)blockIdx.x * THIN_WAVES + wave, nwaves = (int64_t)gridDim.x * THIN_WAVES;
    if (wave_id >= a.units) return;
    const int64_t my_units = (a.units - wave_id + nwaves - 1) / nwaves;
    const int64_t total = my_units * a.groups;        // register sets this wave goes through
    const int chunks = a.kr / Q;                      // whole chunks per row
    Chunk buf[2][THIN_GROUP];
    // the wave's register sets in order: unit after unit (wave_id, wave_id + nwaves, ...), `groups` sets per unit;
    // one cursor for the loads, one for the multiplications behind them
    int64_t u_ld = wave_id, u_mm = wave_id;
    int g_ld = 0, g_mm = 0;
    auto issue = [&](Chunk (&dst)[THIN_GROUP]) __attribute__((always_inline)) {
        const int64_t u = u_ld;
        const int grp = g_ld;
        if (++g_ld == a.groups) {
            g_ld = 0;
            u_ld += nwaves;
        }
        int64_t n = u * THIN_UNIT + j;
        n = n < a.nl ? n : a.nl - 1;                  // (rows past the end read the last row; their results are not stored)
        const R* row = L + n * a.ls_n * nc;
#pragma unroll
        for (int t = 0; t < THIN_GROUP; ++t) {
            const int c = 4 * (grp * THIN_GROUP + t) + g;
            const int cc = c < chunks ? c : chunks - 1;
            // (a cached load: an instruction takes 64 bytes of each of 16 rows, the next one the other half of the same
            // 128-byte lines -- a non-temporal load fetched them twice: 16 rows of 4 KB 964 -> 847 us)
            dst[t] = *(reinterpret_cast<const Chunk*>(row) + cc);
        }
    };
    Acc acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[mb][r] = R(0);
    auto multiply = [&](Chunk (&src)[THIN_GROUP]) __attribute__((always_inline)) {
        const int grp = g_mm;
#pragma unroll
        for (int t = 0; t < THIN_GROUP; ++t) {
            const int i = grp * THIN_GROUP + t;
            Chunk b = src[t];
            if (4 * i + g >= chunks) {                 // a chunk past the row's end (the last set only): nothing
#pragma unroll
                for (int q = 0; q < Q; ++q) b[q] = R(0);
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const Chunk s = As[(mb * steps_p + i) * 64 + lane];
#pragma unroll
                for (int q = 0; q < Q; ++q) acc[mb] = Mfma<R>::run(s[q], b[q], acc[mb]);
            }
        }
    };
    auto finish = [&]() __attribute__((always_inline)) {
        // the unit's results: accumulator r of lane (g, j) is S' row 16 mb + row(lane, r), n = j
        const int64_t u = u_mm;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                tile[j * TP + 16 * mb + Mfma<R>::row(lane, r)] = acc[mb][r];
                acc[mb][r] = R(0);
            }
        thin_wave_sync();
        const int64_t n0 = u * THIN_UNIT;
        const int nn = (int)(a.nl - n0 < THIN_UNIT ? a.nl - n0 : THIN_UNIT);
        R* C = reinterpret_cast<R*>(a.C);
        const int count = a.ms * THIN_UNIT;            // elements of the unit
        if (!a.use_beta) {
            // A fixed number of unconditional stores (lanes past the unit's elements or rows past the end of L write
            // the last element again): the waits for the loads that were issued before them can then count them,
            // instead of waiting for every store of the wave to be acknowledged.
            constexpr int SI = MB * 16 * THIN_UNIT / 64;
#pragma unroll
            for (int it = 0; it < SI; ++it) {
                int e = lane + 64 * it;
                e = e < count ? e : count - 1;
                const int m = a.m_fast ? e % a.ms : e / THIN_UNIT;
                int nl = a.m_fast ? e / a.ms : e % THIN_UNIT;
                nl = nl < nn ? nl : nn - 1;
                R* dst = C + ((int64_t)m * a.cs_m + (n0 + nl) * a.cs_n) * nc;
                if (a.cx) {
                    const double re = tile[nl * TP + 2 * m], im = tile[nl * TP + 2 * m + 1];
                    dst[0] = (R)(a.alpha_re * re - a.alpha_im * im);
                    dst[1] = (R)(a.alpha_re * im + a.alpha_im * re);
                } else {
                    dst[0] = (R)(a.alpha_re * (double)tile[nl * TP + m]);
                }
            }
            thin_wave_sync();
            return;
        }
        for (int e = lane; e < count; e += 64) {
            // m fastest when C is contiguous along m, n fastest otherwise
            const int m = a.m_fast ? e % a.ms : e / THIN_UNIT, nl = a.m_fast ? e / a.ms : e % THIN_UNIT;
            if (nl >= nn) continue;
            R* dst = C + ((int64_t)m * a.cs_m + (n0 + nl) * a.cs_n) * nc;
            if (a.cx) {
                const double re = tile[nl * TP + 2 * m], im = tile[nl * TP + 2 * m + 1];
                double rr = a.alpha_re * re - a.alpha_im * im, ri = a.alpha_re * im + a.alpha_im * re;
                if (a.use_beta) {
                    const double cr = dst[0], ci = dst[1];
                    rr += a.beta_re * cr - a.beta_im * ci;
                    ri += a.beta_re * ci + a.beta_im * cr;
                }
                dst[0] = (R)rr;
                dst[1] = (R)ri;
            } else {
                double v = a.alpha_re * (double)tile[nl * TP + m];
                if (a.use_beta) v += a.beta_re * (double)dst[0];
                dst[0] = (R)v;
            }
        }
        thin_wave_sync();
    };
    auto step = [&](Chunk (&src)[THIN_GROUP]) __attribute__((always_inline)) {
        multiply(src);
        if (g_mm == a.groups - 1) finish();
        if (++g_mm == a.groups) {
            g_mm = 0;
            u_mm += nwaves;
        }
    };
    // Every pass issues its loads whether or not a set is left (past the wave's last unit the loads read the last row
    // of L again): with a fixed number of loads between a set's issue and its use the wait for it can leave the
    // newer ones in flight; a conditional issue makes every wait one for all of them, and loads and MFMAs take turns.
    issue(buf[0]);
    for (int64_t f = 0; f < total; f += 2) {
        issue(buf[1]);
        step(buf[0]);
        if (f + 1 >= total) break;
        issue(buf[0]);
        step(buf[1]);
    }
}

template <class R>
void launch_thin_typed(const ThinArgs& ta, int mb, dim3 grid, size_t lds, hipStream_t st) {
    switch (mb) {
        case 1: TFH_LAUNCH_TIMED((gemm_thin_kernel<R, 1>), grid, dim3(THIN_THREADS), lds, st, ta); break;
        default: TFH_LAUNCH_TIMED((gemm_thin_kernel<R, 2>), grid, dim3(THIN_THREADS), lds, st, ta); break;
    }
}

template <class R>
void raise_thin_lds() {
    const int cap = 160 * 1024;
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_thin_kernel<R, 1>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_thin_kernel<R, 2>), hipFuncAttributeMaxDynamicSharedMemorySize, cap);
}

}  // namespace

// Returns true when the kernel was launched (status holds the outcome).  Takes the products that the register-resident
// streaming kernel does not: more than 32 16-byte chunks of k against at most 32 real rows.
bool try_thin_stream(int dtype, const void* a, const void* b, void* c, const ContractAxes& ax0, Scalar alpha, Scalar beta, void* stream,
                     bool conj_a, bool conj_b, int32_t& status) {
    status = TFH_OK;
    if (!ax0.batch.empty() || ax0.M.empty() || ax0.N.empty() || ax0.K.empty()) return false;
    ContractAxes ax = ax0;
    auto by_c = [](std::vector<Axis>& v) {
        std::stable_sort(v.begin(), v.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[2]) > std::llabs(y.s[2]); });
    };
    by_c(ax.M);
    by_c(ax.N);
    std::stable_sort(ax.K.begin(), ax.K.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[0]) > std::llabs(y.s[0]); });
    fuse_axes(ax.M, 3);
    fuse_axes(ax.N, 3);
    fuse_axes(ax.K, 3);
    if (ax.M.size() != 1 || ax.N.size() != 1 || ax.K.size() != 1) return false;
    const bool cx = is_complex(dtype), dbl = is_double(dtype);
    const int nc = cx ? 2 : 1, q = dbl ? 2 : 4, rb = dbl ? 8 : 4;
    // which side is the small one
    Axis m = ax.M[0], n = ax.N[0], k = ax.K[0];
    const void *S = a, *L = b;
    bool conj_s = conj_a, conj_l = conj_b;
    int slot_s = 0, slot_l = 1;
    if (m.n > n.n) {
        std::swap(m, n);
        std::swap(S, L);
        std::swap(conj_s, conj_l);
        slot_s = 1;
        slot_l = 0;
    }
    const int64_t mr = m.n * nc, kr = k.n * nc;
    // (from 33 real rows on, the matrix cores bound the product more tightly than HBM does -- 64 rows in double precision
    // are 16 flops per byte -- and 128 x 64 tiles use them better: 64 x 64 against a million rows 261 us on tiles, 319 here)
    if (mr > 32 || mr < 2 || n.n < 4096 || k.n < 2) return false;
    const int64_t chunks = kr / q;
    if (kr % q != 0) return false;                                    // rows of L hold whole 16-byte chunks
    if (mr <= 32 && chunks <= 32) return false;                       // the register-resident kernel's
    if (k.s[slot_l] != 1 || n.s[slot_l] < k.n) return false;          // rows of L contiguous in k, one after the other
    if ((n.s[slot_l] * nc) % q != 0 || (uintptr_t)L % 16 != 0) return false;   // ... and starting on 16-byte boundaries
    if (m.s[2] != 1 && n.s[2] != 1) return false;
    if (m.s[slot_s] < 0 || k.s[slot_s] < 0 || m.s[2] <= 0 || n.s[2] <= 0) return false;
    const int mb = (int)((mr + 15) / 16);
    // A small operand over 64 KB goes in passes over slices of k, one launch each on the same stream: the first applies
    // beta, the later ones add to C (C is the small side of the traffic: 32 columns against k = 512 move it three times
    // instead of once, 12 % more bytes).  A slice is a whole number of register sets of chunk steps.
    const int64_t set_chunks = 4 * THIN_GROUP;                                  // chunks per register set and row
    const int64_t max_sets = (int64_t)THIN_S_BYTES / ((int64_t)mb * THIN_GROUP * 64 * 16);
    if (max_sets < 1) return false;
    const int64_t all_sets = (chunks + set_chunks - 1) / set_chunks;
    const int64_t passes = (all_sets + max_sets - 1) / max_sets;
    if (passes > 8) return false;
    const int64_t sets_per_pass = (all_sets + passes - 1) / passes;
    if (n.n > ((int64_t)1 << 40)) return false;
    static const bool raised = [] {
        raise_thin_lds<double>();
        raise_thin_lds<float>();
        return true;
    }();
    (void)raised;
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_CONTRACT, stream);
    for (int64_t pass = 0; pass < passes; ++pass) {
        const int64_t c0 = pass * sets_per_pass * set_chunks, c1 = std::min<int64_t>(chunks, c0 + sets_per_pass * set_chunks);
        if (c0 >= c1) break;
        const int64_t kr0 = c0 * q, krn = (c1 - c0) * q;                          // the slice in reals, in elements: / nc
        const int64_t steps = (c1 - c0 + 3) / 4, groups = (steps + THIN_GROUP - 1) / THIN_GROUP;
        const size_t s_bytes = (size_t)mb * groups * THIN_GROUP * 64 * 16;
        ThinArgs ta;
        std::memset(&ta, 0, sizeof ta);
        ta.S = (const char*)S + (kr0 / nc) * k.s[slot_s] * (int64_t)dtype_size(dtype);
        ta.L = (const char*)L + kr0 * rb;
        ta.C = c;
        ta.ms = (int32_t)m.n;
        ta.K = (int32_t)(krn / nc);
        ta.mr = (int32_t)mr;
        ta.kr = (int32_t)krn;
        ta.steps = (int32_t)steps;
        ta.groups = (int32_t)groups;
        ta.cx = cx;
        ta.conj_s = conj_s && cx;
        ta.conj_l = conj_l && cx;
        ta.use_beta = pass > 0 || !beta.is_zero();
        ta.m_fast = m.s[2] == 1 && n.s[2] != 1;
        ta.nl = n.n;
        ta.units = (n.n + THIN_UNIT - 1) / THIN_UNIT;
        ta.ss_m = m.s[slot_s];
        ta.ss_k = k.s[slot_s];
        ta.ls_n = n.s[slot_l];
        ta.cs_m = m.s[2];
        ta.cs_n = n.s[2];
        ta.alpha_re = alpha.re; ta.alpha_im = alpha.im;
        ta.beta_re = pass > 0 ? 1.0 : beta.re;
        ta.beta_im = pass > 0 ? 0.0 : beta.im;
        const size_t lds = s_bytes + (size_t)THIN_WAVES * THIN_UNIT * (mb * 16 + 1) * rb;
        const int64_t per_cu = lds <= 78 * 1024 ? 2 : 1;   // blocks that fit a CU's 160 KB of LDS
        const int64_t blocks = std::min<int64_t>((ta.units + THIN_WAVES - 1) / THIN_WAVES, 256 * per_cu);
        if (dbl) launch_thin_typed<double>(ta, mb, dim3((uint32_t)blocks), lds, st);
        else launch_thin_typed<float>(ta, mb, dim3((uint32_t)blocks), lds, st);
    }
    prof_end(prof, stream);
    status = hip_check(hipGetLastError(), "contraction kernel launch");
    return true;
}

}  // namespace tfh
