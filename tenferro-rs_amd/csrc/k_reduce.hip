// k_reduce.hip -- multi-axis strided reduction for gfx950: PrimDescriptor::Reduce
// (tenferro-prims/src/lib.rs:170-180), C[kept] = alpha*reduce_op(A[kept, reduced]) + beta*C.
//
// The 256 threads of a block tile the axes that are fastest in A's memory (kept or reduced alike), so
// every wave reads contiguous runs.  A thread walks the remaining reduced extent serially (odometer,
// no division in the loop), lanes that share an output combine through an LDS tree over the thread-id
// bits that belong to reduced axes, and the lanes whose reduced bits are zero write the output.
// When few outputs meet a long reduction the reduced range is split over blockIdx.y into partial
// results that a second small kernel folds in a fixed order (deterministic, no atomics).
// HBM-bound: algorithmic bytes = (input elements + output elements) * sizeof(T).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "internal.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

constexpr int MAXT = 4;
constexpr int MAXG = 16;
constexpr int MAXR = 4;  // serial (outer) reduced axes
constexpr int THREADS = 256;

struct ReduceArgs {
    const void* in;
    const void* in_b;      // second operand of a product reduction (DOT), addressed through t_sb / g_sb / r_sb
    void* out;
    double* partial;       // [nchunks][kept_slots] accumulators (complex: 2 doubles each)
    int32_t nt, ng, nr;
    int32_t tile_elems;
    int32_t red_bits;      // thread-id bits owned by reduced tile axes
    int32_t op;
    int32_t nchunks;
    int32_t use_beta;
    // thread tile, in A-memory order
    int32_t t_shift[MAXT], t_mask[MAXT], t_red[MAXT];
    int64_t t_sa[MAXT], t_sc[MAXT], t_n[MAXT], t_sb[MAXT];
    // kept outer axes -> blockIdx.x
    int64_t g_count[MAXG], g_sa[MAXG], g_sc[MAXG], g_sb[MAXG];
    int32_t g_tid[MAXG], g_text[MAXG];
    // serial reduced axes (innermost first)
    int64_t r_count[MAXR], r_sa[MAXR], r_n[MAXR], r_sb[MAXR];
    int32_t r_tid[MAXR], r_text[MAXR];
    int64_t r_total;       // product of r_count
    int64_t kept_slots;    // gridDim.x * kept lanes per block
    double alpha_re, alpha_im, beta_re, beta_im;
};

__device__ __forceinline__ double combine(double a, double b, int op) {
    return op == TFH_REDUCE_SUM ? a + b : (op == TFH_REDUCE_MAX ? fmax(a, b) : fmin(a, b));
}
__device__ __forceinline__ double identity(int op) {
    return op == TFH_REDUCE_SUM ? 0.0 : (op == TFH_REDUCE_MAX ? -INFINITY : INFINITY);
}

struct ThreadPos {
    int64_t in, out;      // element offsets of this thread (block origin + in-tile position)
    int64_t in_b;         // ... in the second operand of a product reduction
    int64_t lim[MAXT];    // remaining extent of each tile axis at this block
    int32_t tc[MAXT];     // in-tile coordinate per tile axis
    bool ok;              // inside the tensor on every kept tile axis
    bool red_ok;          // inside the tensor on every reduced tile axis
    int32_t kept_lane;    // index of this thread among the block's kept lanes
    bool writer;          // reduced bits all zero
};

__device__ __forceinline__ ThreadPos thread_pos(const ReduceArgs& a, int tid) {
    ThreadPos p;
    p.in = p.out = p.in_b = 0;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) p.lim[t] = t < a.nt ? a.t_n[t] : 1;
    uint64_t bid = blockIdx.x;
    for (int g = 0; g < a.ng; ++g) {
        uint64_t q = bid / (uint64_t)a.g_count[g];
        int64_t c = (int64_t)(bid - q * (uint64_t)a.g_count[g]);
        bid = q;
        p.in += c * a.g_sa[g];
        p.in_b += c * a.g_sb[g];
        p.out += c * a.g_sc[g];
        int t = a.g_tid[g];
#pragma unroll
        for (int k = 0; k < MAXT; ++k)
            if (k == t) p.lim[k] -= c * a.g_text[g];
    }
    p.ok = tid < a.tile_elems;
    p.writer = true;
    p.red_ok = true;
    p.kept_lane = 0;
    int kshift = 0;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) {
        p.tc[t] = 0;
        if (t < a.nt) {
            int c = (tid >> a.t_shift[t]) & a.t_mask[t];
            p.tc[t] = c;
            p.in += (int64_t)c * a.t_sa[t];
            p.in_b += (int64_t)c * a.t_sb[t];
            if (a.t_red[t]) {
                p.writer &= c == 0;
                p.red_ok &= c < a.t_n[t];
            } else {
                p.out += (int64_t)c * a.t_sc[t];
                p.ok &= c < p.lim[t];
                p.kept_lane |= c << kshift;
                kshift += __popc(a.t_mask[t]);
            }
        }
    }
    return p;
}

// DOT: the reduced quantity is the product A * B of two operands read at the same coordinates (sum only).
template <class R, bool CX, bool DOT = false>
__global__ void __launch_bounds__(THREADS) reduce_kernel(ReduceArgs a) {
    prefetch_kernel_arguments<sizeof(ReduceArgs)>();
    constexpr int NC = CX ? 2 : 1;
    __shared__ double lds[THREADS * NC];
    const ThreadPos p = thread_pos(a, threadIdx.x);
    const R* A = reinterpret_cast<const R*>(a.in) + p.in * NC;
    const R* B = DOT ? reinterpret_cast<const R*>(a.in_b) + p.in_b * NC : nullptr;
    const int op = DOT ? (int)TFH_REDUCE_SUM : a.op;   // (a product reduction is always a sum: the selects fold away)
    double acc_re = identity(op), acc_im = 0.0;
    // this block's slice of the serial reduced range
    const int64_t per = (a.r_total + a.nchunks - 1) / a.nchunks;
    const int64_t it0 = (int64_t)blockIdx.y * per;
    const int64_t it1 = it0 + per < a.r_total ? it0 + per : a.r_total;
    // odometer start
    int64_t c[MAXR];
    int64_t off = 0, off_b = 0;
    {
        int64_t lin = it0;
#pragma unroll
        for (int r = 0; r < MAXR; ++r) {
            c[r] = 0;
            if (r < a.nr) {
                int64_t q = lin / a.r_count[r];
                c[r] = lin - q * a.r_count[r];
                lin = q;
                off += c[r] * a.r_sa[r];
                if (DOT) off_b += c[r] * a.r_sb[r];
            }
        }
    }
    // in-tile coordinate of this thread along the tile axis each serial axis extends (0 if none)
    int64_t tcr[MAXR];
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
        tcr[r] = 0;
        if (r < a.nr) {
            int t = a.r_tid[r];
#pragma unroll
            for (int k = 0; k < MAXT; ++k)
                if (k == t) tcr[r] = p.tc[k];
        }
    }
    const bool load_ok = p.ok && p.red_ok;
    constexpr int U = 8;  // independent loads in flight per thread
    for (int64_t it = it0; it < it1; it += U) {
        int64_t offs[U], offs_b[U];
        bool oks[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            bool ok = load_ok && it + u < it1;
#pragma unroll
            for (int r = 0; r < MAXR; ++r)
                if (r < a.nr) ok &= c[r] * a.r_text[r] + tcr[r] < a.r_n[r];
            oks[u] = ok;
            offs[u] = off;
            offs_b[u] = off_b;
            // advance the odometer
            off += a.r_sa[0];
            if (DOT) off_b += a.r_sb[0];
            if (++c[0] == a.r_count[0]) {
                off -= a.r_sa[0] * a.r_count[0];
                if (DOT) off_b -= a.r_sb[0] * a.r_count[0];
                c[0] = 0;
#pragma unroll
                for (int r = 1; r < MAXR; ++r) {
                    if (r < a.nr) {
                        off += a.r_sa[r];
                        if (DOT) off_b += a.r_sb[r];
                        if (++c[r] < a.r_count[r]) break;
                        off -= a.r_sa[r] * a.r_count[r];
                        if (DOT) off_b -= a.r_sb[r] * a.r_count[r];
                        c[r] = 0;
                    }
                }
            }
        }
        R vre[U], vim[U], wre[U], wim[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            vre[u] = vim[u] = wre[u] = wim[u] = R(0);
            if (oks[u]) {
                vre[u] = A[offs[u] * NC];
                if (CX) vim[u] = A[offs[u] * NC + 1];
                if (DOT) {
                    wre[u] = B[offs_b[u] * NC];
                    if (CX) wim[u] = B[offs_b[u] * NC + 1];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (oks[u]) {
                if (DOT) {
                    const double ar = (double)vre[u], ai = (double)vim[u], br = (double)wre[u], bi = (double)wim[u];
                    acc_re += CX ? ar * br - ai * bi : ar * br;
                    if (CX) acc_im += ar * bi + ai * br;
                } else if (CX) {
                    acc_re += (double)vre[u];
                    acc_im += (double)vim[u];
                } else {
                    acc_re = combine(acc_re, (double)vre[u], op);
                }
            }
        }
    }
    // combine lanes that share an output: tree over the reduced thread-id bits
    const int tid = threadIdx.x;
    if (a.red_bits) {
        lds[tid * NC] = acc_re;
        if (CX) lds[tid * NC + 1] = acc_im;
        __syncthreads();
        for (int b = 7; b >= 0; --b) {
            const int bit = 1 << b;
            if (a.red_bits & bit) {
                if (!(tid & bit)) {
                    lds[tid * NC] = combine(lds[tid * NC], lds[(tid | bit) * NC], op);
                    if (CX) lds[tid * NC + 1] += lds[(tid | bit) * NC + 1];
                }
                __syncthreads();
            }
        }
        acc_re = lds[tid * NC];
        if (CX) acc_im = lds[tid * NC + 1];
    }
    if (!(p.writer && p.ok)) return;
    if (a.nchunks > 1) {
        int64_t slot = ((int64_t)blockIdx.y * a.kept_slots + (int64_t)blockIdx.x * THREADS + p.kept_lane) * NC;
        a.partial[slot] = acc_re;
        if (CX) a.partial[slot + 1] = acc_im;
        return;
    }
    R* C = reinterpret_cast<R*>(a.out) + p.out * NC;
    if (CX) {
        double rr = a.alpha_re * acc_re - a.alpha_im * acc_im, ri = a.alpha_re * acc_im + a.alpha_im * acc_re;
        if (a.use_beta) {
            double cr = C[0], ci = C[1];
            rr += a.beta_re * cr - a.beta_im * ci;
            ri += a.beta_re * ci + a.beta_im * cr;
        }
        C[0] = (R)rr;
        C[1] = (R)ri;
    } else {
        double r = a.alpha_re * acc_re;
        if (a.use_beta) r += a.beta_re * (double)C[0];
        C[0] = (R)r;
    }
}

// Second pass of a split reduction: one block per block of the first pass.  The block's kept lanes (thread
// ids whose reduced bits are zero) each own one output; the other threads help: thread (kept lane l, part p)
// folds chunks p, p+P, ... and the parts meet in an LDS tree, so the order of the fold is fixed.
template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) reduce_finalize_kernel(ReduceArgs a) {
    constexpr int NC = CX ? 2 : 1;
    __shared__ double lds[THREADS * NC];
    const int keep_mask = 255 & ~a.red_bits;
    const int kl = 1 << __popc(keep_mask);   // kept lanes per block
    const int P = THREADS / kl;              // helper parts per kept lane
    const int lane = threadIdx.x % kl, part = threadIdx.x / kl;
    // the thread id of kept lane `lane` in the first pass: deposit its bits into the kept bit positions
    int tid0 = 0;
    for (int b = 0, src = 0; b < 8; ++b)
        if (keep_mask >> b & 1) {
            tid0 |= ((lane >> src) & 1) << b;
            ++src;
        }
    const ThreadPos p = thread_pos(a, tid0);
    const int op = a.op;
    double acc_re = identity(op), acc_im = 0.0;
    if (p.ok)
        for (int ch = part; ch < a.nchunks; ch += P) {
            int64_t slot = ((int64_t)ch * a.kept_slots + (int64_t)blockIdx.x * THREADS + p.kept_lane) * NC;
            acc_re = combine(acc_re, a.partial[slot], op);
            if (CX) acc_im += a.partial[slot + 1];
        }
    lds[threadIdx.x * NC] = acc_re;
    if (CX) lds[threadIdx.x * NC + 1] = acc_im;
    __syncthreads();
    for (int step = P >> 1; step > 0; step >>= 1) {
        if (part < step) {
            const int other = (part + step) * kl + lane;
            lds[threadIdx.x * NC] = combine(lds[threadIdx.x * NC], lds[other * NC], op);
            if (CX) lds[threadIdx.x * NC + 1] += lds[other * NC + 1];
        }
        __syncthreads();
    }
    if (part != 0 || !p.ok) return;
    acc_re = lds[threadIdx.x * NC];
    if (CX) acc_im = lds[threadIdx.x * NC + 1];
    R* C = reinterpret_cast<R*>(a.out) + p.out * NC;
    if (CX) {
        double rr = a.alpha_re * acc_re - a.alpha_im * acc_im, ri = a.alpha_re * acc_im + a.alpha_im * acc_re;
        if (a.use_beta) {
            double cr = C[0], ci = C[1];
            rr += a.beta_re * cr - a.beta_im * ci;
            ri += a.beta_re * ci + a.beta_im * cr;
        }
        C[0] = (R)rr;
        C[1] = (R)ri;
    } else {
        double r = a.alpha_re * acc_re;
        if (a.use_beta) r += a.beta_re * (double)C[0];
        C[0] = (R)r;
    }
}

// ---- fast path ------------------------------------------------------------------------------------------------
// Used when no tile is partial (every tiled extent is a multiple of its tile extent), the thread tile is exactly
// 256 lanes and there are enough outputs to fill the chip.  Per load the vector unit does one 64-bit add: the
// thread's in-tile offset is computed once, the block origin is scalar, and the offsets of the serial reduced
// indices come from a small LDS table built at block start.  VEC elements per load along A's contiguous axis
// (16 bytes); KV: that axis is kept (VEC outputs per lane) rather than reduced (summed in registers).
// KS: consecutive outer kept indices handled by one block, each with its own accumulators, so that short
// reductions still give every thread >= 8 independent loads and one LDS tree serves them all.
constexpr int FAST_MAX_RTAB = 1024;
struct FastReduceArgs {
    const void* in;
    void* out;
    int32_t nt, ng, nr, op;
    int32_t red_bits, use_beta;
    int32_t t_shift[MAXT], t_mask[MAXT], t_red[MAXT];
    int64_t t_sa[MAXT], t_sc[MAXT];
    int64_t g_count[MAXG], g_sa[MAXG], g_sc[MAXG];
    int64_t r_count[MAXR], r_sa[MAXR];
    int32_t r_total;
    // >= 0: the blocks of group (blockIdx.x >> rot_shift) start their serial range at index group % r_total and wrap
    // round (mode 0 only); < 0: every block starts at index 0
    int32_t rot_shift;
    int64_t ks_sa, ks_sc;     // strides of the block-serial kept axis
    int32_t bf_bit[3];        // BF: the three lowest reduced thread-id bits inside a wave
    // few outputs, long serial range: blockIdx.y takes `rps` serial indices and writes raw partial results (mode 1),
    // a second launch folds the nchunks partials of every output in a fixed order (mode 2); mode 0: no split
    int32_t mode;
    int32_t nchunks, rps, nblocks;
    double* partial;          // [nchunks][nblocks][THREADS][NV]
    int64_t vc_stride;        // C stride between the VEC outputs of one lane (KV)
    double alpha, beta;
    // floor(2^32 / n) for every grid count and for r_total: division by a launch constant as a multiply-high and one
    // correction step on the scalar unit (a 32-bit division costs ~25 vector instructions in every wave, and with eight
    // blocks per CU all starting at once every instruction before the first load is time the memory system idles)
    uint32_t g_magic[MAXG], rot_magic;
};
// n >= 1, x < 2^32: the quotient estimate mulhi(x, floor(2^32 / n)) is the quotient or one less
__device__ __forceinline__ uint32_t div_magic(uint32_t x, uint32_t n, uint32_t magic, uint32_t& rem) {
    uint32_t q = __umulhi(x, magic);
    rem = x - q * n;
    if (rem >= n) {
        ++q;
        rem -= n;
    }
    return q;
}

template <class R, int N>
struct alignas(sizeof(R) * N) RVec {
    R v[N];
};
template <class R, int N> struct RawV { typedef R type __attribute__((ext_vector_type(N))); };
template <class R> struct RawV<R, 1> { typedef R type; };
// The input is read exactly once: non-temporal loads (a read-only sweep of 134 MB measures 6.7 TB/s with the hint
// against 6.3 TB/s without on this device).
template <class R, int N>
__device__ __forceinline__ RVec<R, N> load_stream(const R* p) {
    typedef typename RawV<R, N>::type Raw;
    return __builtin_bit_cast(RVec<R, N>, __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p)));
}

// SUM: the operation is known to be a sum (otherwise it is a.op at run time, and every element pays for an add, a
// max, a min and the selects between them: ten f64 instructions per 16 bytes loaded instead of two)
template <class R, int VEC, bool KV, int KS, bool BF, bool SUM = false>
__global__ void __launch_bounds__(THREADS) reduce_fast_kernel(FastReduceArgs a) {
    prefetch_kernel_arguments<sizeof(FastReduceArgs)>();
    constexpr int NV = KV ? VEC : 1;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    int64_t* rtab = reinterpret_cast<int64_t*>(smem_raw);                               // [r_total]
    double* lds = reinterpret_cast<double*>(smem_raw + FAST_MAX_RTAB * sizeof(int64_t)); // [KS*NV][THREADS]
    const int tid = threadIdx.x;
    const int r_begin = a.mode == 1 ? (int)blockIdx.y * a.rps : 0;
    const int r_count = a.mode == 2 ? 0 : (a.mode == 1 ? (a.r_total - r_begin < a.rps ? a.r_total - r_begin : a.rps) : a.r_total);
    // (a split reduction rotates every chunk by its own number: the chunks run in step as well, a power of two apart)
    int rot = 0;
    if (a.rot_shift >= 0 && a.mode == 0) {
        uint32_t rem;
        (void)div_magic(blockIdx.x >> a.rot_shift, (uint32_t)r_count, a.rot_magic, rem);
        rot = (int)rem;
    }
    if (a.mode == 1 && r_count > 0) rot = (int)(blockIdx.y % (uint32_t)r_count);
    for (int i = tid; i < r_count; i += THREADS) {
        // (the serial range is at most FAST_MAX_RTAB long: 32-bit arithmetic, and the outermost axis takes what is left)
        uint32_t lin = (uint32_t)(r_begin + (i + rot >= r_count ? i + rot - r_count : i + rot));
        int64_t off = 0;
#pragma unroll
        for (int r = 0; r < MAXR; ++r)
            if (r < a.nr) {
                if (r + 1 < a.nr) {
                    const uint32_t n = (uint32_t)a.r_count[r], q = lin / n;
                    off += (int64_t)(lin - q * n) * a.r_sa[r];
                    lin = q;
                } else {
                    off += (int64_t)lin * a.r_sa[r];
                }
            }
        rtab[i] = off;
    }
    // block origin (uniform) and this thread's offsets inside the tile
    int64_t org_in = 0, org_out = 0;
    {
        uint32_t bid = blockIdx.x;   // the grid (and so every count) is below 2^31
        for (int g = 0; g < a.ng; ++g) {
            uint32_t c;
            bid = div_magic(bid, (uint32_t)a.g_count[g], a.g_magic[g], c);
            org_in += (int64_t)c * a.g_sa[g];
            org_out += (int64_t)c * a.g_sc[g];
        }
    }
    int64_t toff_in = 0, toff_out = 0;
    bool writer = true;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) {   // unused slots are neutral (mask 0)
        const int c = (tid >> a.t_shift[t]) & a.t_mask[t];
        toff_in += (int64_t)c * a.t_sa[t];
        if (a.t_red[t]) writer &= c == 0;
        else toff_out += (int64_t)c * a.t_sc[t];
    }
    const int op = SUM ? (int)TFH_REDUCE_SUM : a.op;
    __syncthreads();
    const R* A = reinterpret_cast<const R*>(a.in) + org_in + toff_in;
    double acc[KS][NV];
#pragma unroll
    for (int k = 0; k < KS; ++k)
#pragma unroll
        for (int j = 0; j < NV; ++j) acc[k][j] = identity(op);
    constexpr int U = KS >= 8 ? 2 : 8;
    // a rolling window of U loads per thread: the load of step it+U is issued as soon as the value of step it has
    // been taken, so the memory pipeline never drains between batches
#pragma unroll
    for (int k = 0; k < KS; ++k) {
        const R* Ak = A + k * a.ks_sa;
        RVec<R, VEC> v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (u < r_count) v[u] = load_stream<R, VEC>(Ak + rtab[u]);
        for (int it = 0; it < r_count; it += U) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (it + u >= r_count) break;
                const RVec<R, VEC> x = v[u];
                if (it + U + u < r_count) v[u] = load_stream<R, VEC>(Ak + rtab[it + U + u]);
                if (KV) {
#pragma unroll
                    for (int j = 0; j < VEC; ++j) acc[k][j] = combine(acc[k][j], (double)x.v[j], op);
                } else {
                    double s = (double)x.v[0];
#pragma unroll
                    for (int j = 1; j < VEC; ++j) s = combine(s, (double)x.v[j], op);
                    acc[k][0] = combine(acc[k][0], s, op);
                }
            }
        }
    }
    if (KS == 1 && a.mode == 2) {
        // second launch of a split reduction: the lanes that share an output take the partials of the chunks in turn
        // (chunk = the lane's reduced bits, compressed, then every P-th) and the ordinary fold below adds them up
        int part = 0, P = 1;
        for (int b = 0; b < 8; ++b)
            if (a.red_bits & (1 << b)) {
                part |= ((tid >> b) & 1) * P;
                P <<= 1;
            }
        const int wl = tid & ~a.red_bits;
        for (int ch = part; ch < a.nchunks; ch += P) {
            const double* src = a.partial + (((int64_t)ch * a.nblocks + blockIdx.x) * THREADS + wl) * NV;
#pragma unroll
            for (int j = 0; j < NV; ++j) acc[0][j] = combine(acc[0][j], src[j], op);
        }
    }
    if constexpr (BF) {
        // Eight accumulators per lane, every lane of a group holding a partial sum of each: a transposing butterfly.
        // Across reduced bit b0 a lane keeps the four accumulators whose index has its own bit value in place 0 and
        // hands the other four to its partner, then the same with two across b1 and one across b2 -- seven exchanges
        // instead of twenty-four, after which the lane owns the output with index (its bits b0, b1, b2) and only
        // that one value goes through the rest of the fold.
        static_assert(KS == 8, "the butterfly folds eight block-serial outputs");
        const int m0 = (tid >> a.bf_bit[0]) & 1, m1 = (tid >> a.bf_bit[1]) & 1, m2 = (tid >> a.bf_bit[2]) & 1;
        const int x0 = 1 << a.bf_bit[0], x1 = 1 << a.bf_bit[1], x2 = 1 << a.bf_bit[2];
        double one[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            double a4[4], a2[2];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const double keep = m0 ? acc[2 * q + 1][j] : acc[2 * q][j], send = m0 ? acc[2 * q][j] : acc[2 * q + 1][j];
                a4[q] = combine(keep, __shfl_xor(send, x0), op);
            }
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                const double keep = m1 ? a4[2 * q + 1] : a4[2 * q], send = m1 ? a4[2 * q] : a4[2 * q + 1];
                a2[q] = combine(keep, __shfl_xor(send, x1), op);
            }
            const double keep = m2 ? a2[1] : a2[0], send = m2 ? a2[0] : a2[1];
            one[j] = combine(keep, __shfl_xor(send, x2), op);
        }
        const int rest = a.red_bits & ~(x0 | x1 | x2);
#pragma unroll
        for (int b = 0; b < 6; ++b)
            if (rest & (1 << b)) {
#pragma unroll
                for (int j = 0; j < NV; ++j) one[j] = combine(one[j], __shfl_xor(one[j], 1 << b), op);
            }
        if (rest & 0xc0) {
#pragma unroll
            for (int j = 0; j < NV; ++j) lds[j * THREADS + tid] = one[j];
            __syncthreads();
            for (int b = 7; b >= 6; --b) {
                const int bit = 1 << b;
                if (rest & bit) {
                    if (!(tid & bit)) {
#pragma unroll
                        for (int j = 0; j < NV; ++j) lds[j * THREADS + tid] = combine(lds[j * THREADS + tid], lds[j * THREADS + (tid | bit)], op);
                    }
                    __syncthreads();
                }
            }
#pragma unroll
            for (int j = 0; j < NV; ++j) one[j] = lds[j * THREADS + tid];
        }
        if ((tid & rest) == 0) {
            const int k = m0 + 2 * m1 + 4 * m2;
            R* C = reinterpret_cast<R*>(a.out) + org_out + toff_out + k * a.ks_sc;
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                R* dst = C + j * a.vc_stride;
                double r = a.alpha * one[j];
                if (a.use_beta) r += a.beta * (double)*dst;
                *dst = (R)r;
            }
        }
        return;
    }
    // lanes that share outputs fold over the reduced thread-id bits: inside a wave with lane exchanges, across
    // waves (bits 6 and 7) through LDS
#pragma unroll
    for (int b = 0; b < 6; ++b)
        if (a.red_bits & (1 << b)) {
#pragma unroll
            for (int k = 0; k < KS; ++k)
#pragma unroll
                for (int j = 0; j < NV; ++j) acc[k][j] = combine(acc[k][j], __shfl_xor(acc[k][j], 1 << b), op);
        }
    if (a.red_bits & 0xc0) {
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int j = 0; j < NV; ++j) lds[(k * NV + j) * THREADS + tid] = acc[k][j];
        __syncthreads();
        for (int b = 7; b >= 6; --b) {
            const int bit = 1 << b;
            if (a.red_bits & bit) {
                if (!(tid & bit)) {
#pragma unroll
                    for (int q = 0; q < KS * NV; ++q) lds[q * THREADS + tid] = combine(lds[q * THREADS + tid], lds[q * THREADS + (tid | bit)], op);
                }
                __syncthreads();
            }
        }
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int j = 0; j < NV; ++j) acc[k][j] = lds[(k * NV + j) * THREADS + tid];
    }
    if (writer && KS == 1 && a.mode == 1) {
        double* dst = a.partial + (((int64_t)blockIdx.y * a.nblocks + blockIdx.x) * THREADS + tid) * NV;
#pragma unroll
        for (int j = 0; j < NV; ++j) dst[j] = acc[0][j];
        return;
    }
    if (writer) {
        R* C = reinterpret_cast<R*>(a.out) + org_out + toff_out;
#pragma unroll
        for (int k = 0; k < KS; ++k)
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                R* dst = C + k * a.ks_sc + j * a.vc_stride;
                double r = a.alpha * acc[k][j];
                if (a.use_beta) r += a.beta * (double)*dst;
                *dst = (R)r;
            }
    }
}

template <class R, int VEC, bool KV, bool SUM>
void launch_fast_op(const FastReduceArgs& fa, dim3 grid, int ks, bool bf, hipStream_t st) {
    const int nv = KV ? VEC : 1;
    if (ks == 8 && bf) {
        size_t lds = FAST_MAX_RTAB * sizeof(int64_t) + (size_t)nv * THREADS * sizeof(double);
        TFH_LAUNCH_TIMED((reduce_fast_kernel<R, VEC, KV, 8, true, SUM>), grid, dim3(THREADS), lds, st, fa);
    } else if (ks == 8) {
        size_t lds = FAST_MAX_RTAB * sizeof(int64_t) + (size_t)8 * nv * THREADS * sizeof(double);
        TFH_LAUNCH_TIMED((reduce_fast_kernel<R, VEC, KV, 8, false, SUM>), grid, dim3(THREADS), lds, st, fa);
    } else {
        size_t lds = FAST_MAX_RTAB * sizeof(int64_t) + (size_t)nv * THREADS * sizeof(double);
        TFH_LAUNCH_TIMED((reduce_fast_kernel<R, VEC, KV, 1, false, SUM>), grid, dim3(THREADS), lds, st, fa);
    }
}
template <class R, int VEC, bool KV>
void launch_fast_ks(const FastReduceArgs& fa, dim3 grid, int ks, bool bf, hipStream_t st) {
    if (fa.op == TFH_REDUCE_SUM) launch_fast_op<R, VEC, KV, true>(fa, grid, ks, bf, st);
    else launch_fast_op<R, VEC, KV, false>(fa, grid, ks, bf, st);
}
template <class R>
void launch_fast(const FastReduceArgs& fa, dim3 grid, int vec, bool kv, int ks, bool bf, hipStream_t st) {
    constexpr int V = 16 / sizeof(R);
    if (vec > 1) {
        if (kv) launch_fast_ks<R, V, true>(fa, grid, ks, bf, st);
        else launch_fast_ks<R, V, false>(fa, grid, ks, bf, st);
    } else
        launch_fast_ks<R, 1, true>(fa, grid, ks, bf, st);
}

int ceil_log2(int64_t n) {
    int l = 0;
    while (((int64_t)1 << l) < n) ++l;
    return l;
}

}  // namespace

namespace {
// Returns true when the fast kernel was launched.
bool try_fast_reduce(int dtype, const void* a, void* c, std::vector<Axis> kept, std::vector<Axis> red, int reduce_op,
                     Scalar alpha, Scalar beta, void* stream, int32_t& status) {
    status = TFH_OK;
    const bool cx = is_complex(dtype);
    if (cx && (reduce_op != TFH_REDUCE_SUM || alpha.im != 0 || beta.im != 0)) return false;
    const int rbytes = is_double(dtype) ? 8 : 4;
    if (cx) {   // complex sum = real sum over the interleaved layout with an extra kept axis (re, im)
        for (auto& x : kept) { x.s[0] *= 2; x.s[1] *= 2; }
        for (auto& x : red) x.s[0] *= 2;
        kept.push_back(Axis{2, {1, 1, 0}, 0xffffffffu});
    }
    std::stable_sort(kept.begin(), kept.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    for (auto& x : kept) x.s[2] = 0;
    fuse_axes(kept, 2);
    for (auto& x : red) x.s[1] = x.s[2] = 0;
    std::stable_sort(red.begin(), red.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[0]) > std::llabs(y.s[0]); });
    fuse_axes(red, 1);
    for (auto& x : kept)
        if (x.s[1] == 0 || x.s[0] == 0) return false;
    for (auto& x : red)
        if (x.s[0] == 0) return false;
    struct Ax { Axis a; bool red; int tl; int64_t neff; };
    std::vector<Ax> all;
    for (auto& x : kept) all.push_back({x, false, 0, x.n});
    for (auto& x : red) all.push_back({x, true, 0, x.n});
    if (all.empty() || (int)all.size() > MAXG) return false;
    std::stable_sort(all.begin(), all.end(), [](const Ax& x, const Ax& y) { return std::llabs(x.a.s[0]) < std::llabs(y.a.s[0]); });
    // vector loads along A's contiguous axis
    int vec = 16 / rbytes;
    {
        Ax& f = all[0];
        bool ok = f.a.s[0] == 1 && f.a.n % vec == 0 && ((uintptr_t)a % 16) == 0;
        for (size_t i = 1; i < all.size(); ++i) ok &= all[i].a.s[0] % vec == 0;
        if (!ok) vec = 1;
    }
    const bool kv = !all[0].red;
    all[0].neff = all[0].a.n / vec;
    FastReduceArgs fa;
    std::memset(&fa, 0, sizeof fa);
    int bits = 8, shift = 0;
    for (size_t i = 0; i < all.size(); ++i) {
        Ax& x = all[i];
        if (bits == 0) break;
        int t = std::min(ceil_log2(x.neff), bits);
        while (t > 0 && x.neff % ((int64_t)1 << t) != 0) --t;   // no partial tiles
        if (t == 0) {
            if (x.neff == 1) continue;
            break;   // an odd extent blocks the tile: not a fast-path shape
        }
        if (fa.nt == MAXT) break;
        x.tl = t;
        const int id = fa.nt++;
        const int64_t mul = i == 0 ? vec : 1;
        fa.t_shift[id] = shift;
        fa.t_mask[id] = (1 << t) - 1;
        fa.t_red[id] = x.red;
        fa.t_sa[id] = x.a.s[0] * mul;
        fa.t_sc[id] = x.a.s[1] * mul;
        if (x.red) fa.red_bits |= fa.t_mask[id] << shift;
        shift += t;
        bits -= t;
    }
    if (bits != 0) return false;
    {
        // the contiguous bytes that a tile reads at a stretch: a tile that takes two reals of every row of 66 (an odd
        // extent behind a factor of two) uses 8 bytes of every 64 fetched -- the dense-run kernels take such shapes
        int64_t run = 1;
        bool cut = false;   // the stretch ends inside an axis that goes on in memory
        for (size_t i = 0; i < all.size(); ++i) {
            const Ax& x = all[i];
            const int64_t mul = i == 0 ? vec : 1;
            if (std::llabs(x.a.s[0]) != run) break;
            run *= ((int64_t)1 << x.tl) * mul;
            if (((int64_t)1 << x.tl) * mul != x.a.n) {
                cut = true;
                break;
            }
        }
        if (cut && run * rbytes < 64) return false;
    }
    int64_t blocks = 1, r_total = 1;
    for (size_t i = 0; i < all.size(); ++i) {
        const Ax& x = all[i];
        const int64_t text = (int64_t)1 << x.tl;
        const int64_t cnt = x.neff / text;
        if (cnt <= 1) continue;
        const int64_t mul = (i == 0 ? vec : 1) * text;
        if (x.red) {
            if (fa.nr == MAXR) return false;
            fa.r_count[fa.nr] = cnt;
            fa.r_sa[fa.nr] = x.a.s[0] * mul;
            ++fa.nr;
            r_total *= cnt;
        } else {
            fa.g_count[fa.ng] = cnt;
            fa.g_sa[fa.ng] = x.a.s[0] * mul;
            fa.g_sc[fa.ng] = x.a.s[1] * mul;
            ++fa.ng;
            blocks *= cnt;
        }
    }
    if (blocks > 0x7fffffffll) return false;
    // Few outputs and a long serial range: split the range over blockIdx.y (raw partials, then a second launch folds
    // them) so that the chip is filled; this also lifts the limit of the serial-offset table, which then holds one
    // chunk.
    int64_t nchunks = 1, rps = r_total;
    if ((blocks < 512 && r_total >= 64) || r_total > FAST_MAX_RTAB) {   // (a serial range longer than the offset table is split as well)
        nchunks = std::max<int64_t>(1, std::min<int64_t>((2048 + blocks - 1) / blocks, r_total / 16));
        rps = (r_total + nchunks - 1) / nchunks;
        if (rps > FAST_MAX_RTAB) rps = FAST_MAX_RTAB;
        nchunks = (r_total + rps - 1) / rps;
        if (nchunks > 65535) return false;
    }
    // block-serial kept indices when the serial reduction alone gives a thread too few loads
    int ks = 1;
    const int nv = kv ? vec : 1;
    if (nchunks == 1 && r_total < 8 && fa.ng > 0 && fa.g_count[0] % 8 == 0 && blocks / 8 >= 512 && nv <= 2) {   // nv <= 2: LDS stays under 48 KB
        ks = 8;
        fa.ks_sa = fa.g_sa[0];
        fa.ks_sc = fa.g_sc[0];
        fa.g_count[0] /= 8;
        fa.g_sa[0] *= 8;
        fa.g_sc[0] *= 8;
        blocks /= 8;
    }
    fa.r_total = (int32_t)r_total;
    // A serial axis with a kept axis outside it (sum over a middle axis): the blocks of the launch run in step, so at
    // any moment they would all read the same serial index -- addresses that differ by the outer axis's stride, a large
    // power of two in the usual case, which fall into the same DRAM banks.  Groups of 32 consecutive blocks start at
    // different serial indices instead (the order of a block's additions stays fixed, so results are reproducible).
    // 16^6 f64 summed over axes 1 and 4: 25.2 -> 24.1 us; [16,64,16,1024] over axis 1: 30.2 -> 26.1 us; 32^5 f32 over
    // axis 1: 33.8 -> 29.9 us.  A serial axis that is outermost keeps the plain order: there the blocks sweep one
    // contiguous slab after another, and rotating them measured 2-6 % slower.  A reduction split over blockIdx.y rotates
    // each chunk by its number in the kernel (column sums of 4096^2 f64: 29.1 -> 27.2 us, [1024,128,128] over axis 0:
    // 30.4 -> 26.8 us, never slower).
    fa.rot_shift = -1;
    if (nchunks == 1 && r_total >= 4 && blocks >= 512 && fa.nr >= 1 && fa.ng >= 1) {
        int64_t serial_min = INT64_MAX, grid_max = 0;
        for (int r = 0; r < fa.nr; ++r) serial_min = std::min<int64_t>(serial_min, std::llabs(fa.r_sa[r]));
        for (int g = 0; g < fa.ng; ++g) grid_max = std::max<int64_t>(grid_max, std::llabs(fa.g_sa[g]));
        // (serial steps of at least 32 KB: shorter ones measured within 2 % either way)
        if (grid_max > serial_min && serial_min * rbytes >= 32768) fa.rot_shift = 5;
    }
    auto magic_of = [](int64_t n) { return n <= 1 ? 0xffffffffu : (uint32_t)(((uint64_t)1 << 32) / (uint64_t)n); };
    for (int g = 0; g < fa.ng; ++g) fa.g_magic[g] = magic_of(fa.g_count[g]);
    fa.rot_magic = magic_of(r_total);
    fa.in = a;
    fa.out = c;
    fa.op = reduce_op;
    fa.alpha = alpha.re;
    fa.beta = beta.re;
    fa.use_beta = !beta.is_zero();
    fa.vc_stride = all[0].a.s[1];
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((uint32_t)blocks, (uint32_t)nchunks);
    if (nchunks > 1) {
        void* ws = nullptr;
        if (int32_t e = workspace(stream, (size_t)nchunks * (size_t)blocks * THREADS * nv * sizeof(double), &ws)) {
            status = e;
            return true;
        }
        fa.mode = 1;
        fa.nchunks = (int32_t)nchunks;
        fa.rps = (int32_t)rps;
        fa.nblocks = (int32_t)blocks;
        fa.partial = (double*)ws;
    }
    const int prof = prof_begin(PROF_REDUCE, stream);
    // eight block-serial outputs and at least three reduced lane bits inside a wave: the transposing butterfly
    bool bf = false;
    if (ks == 8) {
        int found = 0;
        for (int b = 0; b < 6 && found < 3; ++b)
            if (fa.red_bits & (1 << b)) fa.bf_bit[found++] = b;
        bf = found == 3;
    }
    if (rbytes == 8) launch_fast<double>(fa, grid, vec, kv, ks, bf, st);
    else launch_fast<float>(fa, grid, vec, kv, ks, bf, st);
    prof_end(prof, stream);
    if (nchunks > 1) {
        fa.mode = 2;
        if (rbytes == 8) launch_fast<double>(fa, dim3((uint32_t)blocks), vec, kv, ks, bf, st);
        else launch_fast<float>(fa, dim3((uint32_t)blocks), vec, kv, ks, bf, st);
    }
    status = hip_check(hipGetLastError(), "reduce kernel launch");
    return true;
}
}  // namespace

// ---- short contiguous rows --------------------------------------------------------------------------------------
// A reduced axis of 2..32 elements that is A's contiguous axis, directly inside a kept axis (a dense [rows][n] matrix
// summed along its short rows: a physical index of 3, a bond of 17).  When the extents tile, the fast kernel spreads
// the row over lanes; when they do not, the general kernel did the same with most lanes idle and a fold per row
// ([100,100,100,17] f64 over the last axis: 510 us, 0.28 TB/s).  Here a block takes 256 rows: their 256 * n elements
// are one contiguous run, read with coalesced loads and parked in LDS (row pitch odd, so the next step has no bank
// conflicts), and every thread then adds up its own row in index order and writes one output.
struct ShortRowArgs {
    const void* in;
    void* out;
    int32_t n, pitch;          // row length, LDS row pitch (n, or n + 1 when n is even)
    int32_t op, use_beta, ng;
    int64_t rows, sc;          // extent of the kept axis the rows belong to (A stride n) and its C stride
    int64_t g_count[MAXG], g_sa[MAXG], g_sc[MAXG];   // [0]: blocks of 256 rows; then the outer kept axes
    double alpha, beta;
};

template <class R>
__global__ void __launch_bounds__(THREADS) reduce_shortrow_kernel(ShortRowArgs a) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    R* lds = reinterpret_cast<R*>(smem_raw);
    const int tid = threadIdx.x;
    uint32_t bid = blockIdx.x;
    const uint32_t nrb = (uint32_t)a.g_count[0], rb = bid % nrb;
    bid /= nrb;
    int64_t org_in = 0, org_out = 0;
    for (int g = 1; g < a.ng; ++g) {
        const uint32_t cnt = (uint32_t)a.g_count[g], q = bid / cnt;
        const int64_t c = (int64_t)(bid - q * cnt);
        bid = q;
        org_in += c * a.g_sa[g];
        org_out += c * a.g_sc[g];
    }
    const int64_t row0 = (int64_t)rb * THREADS;
    const int nrows = (int)(a.rows - row0 < THREADS ? a.rows - row0 : THREADS);
    const int n = a.n, pitch = a.pitch, total = nrows * n;
    const R* A = reinterpret_cast<const R*>(a.in) + org_in + row0 * n;
    constexpr int U = 8;   // loads in flight per thread
    for (int j0 = 0; j0 < n; j0 += U) {
        R v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int e = tid + THREADS * (j0 + u);
            if (j0 + u < n && e < total) v[u] = __builtin_nontemporal_load(A + e);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int e = tid + THREADS * (j0 + u);
            if (j0 + u < n && e < total) lds[pitch == n ? e : e + e / n] = v[u];
        }
    }
    __syncthreads();
    if (tid >= nrows) return;
    const int op = a.op;
    double acc = identity(op);
    const R* row = lds + tid * pitch;
    for (int r = 0; r < n; ++r) acc = combine(acc, (double)row[r], op);
    R* dst = reinterpret_cast<R*>(a.out) + org_out + (row0 + tid) * a.sc;
    double res = a.alpha * acc;
    if (a.use_beta) res += a.beta * (double)*dst;
    *dst = (R)res;
}

namespace {
// Returns true when the short-row kernel was launched.
bool try_shortrow_reduce(int dtype, const void* a, void* c, std::vector<Axis> kept, std::vector<Axis> red, int reduce_op,
                         Scalar alpha, Scalar beta, void* stream, int32_t& status) {
    status = TFH_OK;
    if (is_complex(dtype)) return false;
    for (auto& x : red) x.s[1] = x.s[2] = 0;
    std::stable_sort(red.begin(), red.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[0]) > std::llabs(y.s[0]); });
    fuse_axes(red, 1);
    if (red.size() != 1 || red[0].s[0] != 1 || red[0].n < 2 || red[0].n > 32) return false;
    const int64_t n = red[0].n;
    for (auto& x : kept) x.s[2] = 0;
    std::stable_sort(kept.begin(), kept.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    fuse_axes(kept, 2);
    if (kept.empty() || (int)kept.size() > MAXG - 1) return false;
    for (auto& x : kept)
        if (x.s[1] == 0) return false;   // (the general path reports aliasing outputs)
    // the kept axis the rows belong to: the one with A stride n
    size_t ri = kept.size();
    for (size_t i = 0; i < kept.size(); ++i)
        if (kept[i].s[0] == n) ri = i;
    if (ri == kept.size() || kept[ri].n < 1024) return false;
    ShortRowArgs sa;
    std::memset(&sa, 0, sizeof sa);
    sa.in = a;
    sa.out = c;
    sa.n = (int32_t)n;
    sa.pitch = (int32_t)(n | 1);
    sa.op = reduce_op;
    sa.use_beta = !beta.is_zero();
    sa.alpha = alpha.re;
    sa.beta = beta.re;
    sa.rows = kept[ri].n;
    sa.sc = kept[ri].s[1];
    int64_t blocks = (kept[ri].n + THREADS - 1) / THREADS;
    sa.g_count[0] = blocks;
    sa.ng = 1;
    for (size_t i = 0; i < kept.size(); ++i) {
        if (i == ri) continue;
        sa.g_count[sa.ng] = kept[i].n;
        sa.g_sa[sa.ng] = kept[i].s[0];
        sa.g_sc[sa.ng] = kept[i].s[1];
        ++sa.ng;
        blocks *= kept[i].n;
        if (blocks > 0x7fffffffll) return false;
    }
    const size_t lds = (size_t)THREADS * sa.pitch * (is_double(dtype) ? 8 : 4);
    static const bool lds_limit_raised = [] {   // rows of 32 doubles need 66 KB, above the default limit of 64 KB
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&reduce_shortrow_kernel<double>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  THREADS * 33 * 8);
        return true;
    }();
    (void)lds_limit_raised;
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_REDUCE, stream);
    if (is_double(dtype)) TFH_LAUNCH_TIMED((reduce_shortrow_kernel<double>), dim3((uint32_t)blocks), dim3(THREADS), lds, st, sa);
    else TFH_LAUNCH_TIMED((reduce_shortrow_kernel<float>), dim3((uint32_t)blocks), dim3(THREADS), lds, st, sa);
    prof_end(prof, stream);
    status = hip_check(hipGetLastError(), "reduce kernel launch");
    return true;
}
}  // namespace

namespace {
// ---- dense runs of any extent -------------------------------------------------------------------------------------
// For an operand whose fastest axes are dense in memory (any contiguous tensor), whatever the extents are.  A tile is
// a contiguous run of memory: the innermost axes whole, kept and reduced alike, and a range of the next axis, so it
// has one ragged edge at most (the last range of that axis) and no lane idles at an extent that is not a power of
// two.  Thread t owns the 16-byte vectors t, t + 256, ... of the run, whatever coordinates they have, and adds up the
// tiles that the reduced axes outside the tile step through (an odometer of scalar offsets, several tiles' loads in
// flight).  Only when the walk is over do coordinates matter: the accumulators go to LDS and every reduced axis inside
// the tile is folded there, a pass per axis, wide axes in rounds of sixteen so that all threads take part; what is
// left are the tile's outputs in memory order.  A complex element is a kept innermost axis of two reals.  When the
// kept axes outside the tile give too few blocks, the walk is split over blockIdx.y into partial results that a
// second kernel folds in a fixed order.  The loads need only the alignment of a real: a tile starts wherever the
// extents put it.  A vector never reaches past the end of its tile (the last odd reals are read one by one), so
// nothing is read outside the operand.
constexpr int RUN_AXES = 6;        // tile axes, the pair of reals of a complex element included
constexpr int RUN_REALS = 2048;    // accumulators of a tile, parked in LDS as doubles
struct RunArgs {
    const void* in;
    void* out;
    double* partial;               // [nsplit][blocks][kept_per_tile] (complex: 2 doubles each)
    int32_t nf;                    // tile axes in reals, innermost first; the last one is the ranged axis
    int32_t f_ext[RUN_AXES], f_red[RUN_AXES];
    int64_t f_so[RUN_AXES];        // C stride of a kept tile axis, in elements
    int32_t tile_reals;            // product of f_ext
    int32_t row_reals;             // reals per index of the ranged axis
    int32_t kept_per_tile;         // outputs of a full tile
    int32_t range, x_n;            // indices of the ranged axis per tile, and its extent
    int32_t g0_is_range, r0_is_range;   // the tile index along the ranged axis is g[0] (kept) or r[0] (reduced)
    int32_t all_reduced;           // no kept tile axis (a complex element's pair of reals aside)
    int32_t ng, nr;
    int64_t g_count[MAXG], g_si[MAXG], g_so[MAXG];   // kept axes outside the tile (A strides in reals, C in elements)
    int64_t r_count[MAXR], r_si[MAXR];               // reduced axes outside the tile, innermost first
    int64_t r_total, per_split, blocks;
    int32_t nsplit, op, use_beta;
    double alpha_re, alpha_im, beta_re, beta_im;
};

// value known to be the same in every lane -> scalar registers
__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

struct RunOdometer {
    int64_t c[MAXR];
    int64_t off;
};
__device__ __forceinline__ void run_advance(const RunArgs& a, RunOdometer& o) {
    o.off += a.r_si[0];
    if (++o.c[0] == a.r_count[0]) {
        o.off -= a.r_si[0] * a.r_count[0];
        o.c[0] = 0;
#pragma unroll
        for (int r = 1; r < MAXR; ++r) {
            if (r < a.nr) {
                o.off += a.r_si[r];
                if (++o.c[r] < a.r_count[r]) break;
                o.off -= a.r_si[r] * a.r_count[r];
                o.c[r] = 0;
            }
        }
    }
}

template <class R, int NV> struct RunVec { typedef R type __attribute__((ext_vector_type(NV), aligned(sizeof(R)))); };

// UU tiles: all their loads first, then the adds.  A tile of `len` reals is len / NV whole vectors, vector v in slot v
// (thread v % 256, register set v / 256), and up to NV - 1 odd reals behind them, real i of which lane i of the first
// wave adds up in `odd`.  Slots past the tile read the tile's last vector again (an address inside the operand) and
// what they add up is never used.  RAGGED: some of the tiles are shorter than the block's tile (the last range of a
// reduced axis): their slots past the end must stay out of the sums, and their odd reals belong to the accumulators
// of a whole slot.
template <class R, int J, int UU, bool SUM, bool RAGGED>
__device__ __forceinline__ void run_tiles(const RunArgs& a, const R* A, RunOdometer& odo, const int (&own)[J], int len_blk, int op,
                                          double (&acc)[J][16 / sizeof(R)], double& odd) {
    constexpr int NV = 16 / sizeof(R);
    typedef typename RunVec<R, NV>::type V;
    int64_t offs[UU];
    int lens[UU];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        offs[u] = uniform64(odo.off);
        lens[u] = len_blk;
        if (RAGGED) {
            const int64_t left = (int64_t)a.x_n - odo.c[0] * a.range;
            lens[u] = (int)(left < a.range ? left : a.range) * a.row_reals;
        }
        run_advance(a, odo);
    }
    V v[UU][J];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        const int last = lens[u] / NV - 1;   // (a tile shorter than a vector: no slot reads anything it may use)
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const int at = own[j] < last * NV ? own[j] : last * NV;
            v[u][j] = V{};
            if (last >= 0) v[u][j] = __builtin_nontemporal_load(reinterpret_cast<const V*>(A + offs[u] + at));
        }
    }
    // the odd reals behind the block's whole vectors: lane i of the first wave reads real i of them
    const int whole_blk = len_blk / NV * NV, rest_blk = len_blk - whole_blk;
    const bool odd_wave = rest_blk > 0 && threadIdx.x < 64;
    R vo[UU];
    if (odd_wave) {
        const int at = whole_blk + ((int)threadIdx.x < rest_blk ? (int)threadIdx.x : rest_blk - 1);
#pragma unroll
        for (int u = 0; u < UU; ++u) {
            vo[u] = R(0);
            if (!RAGGED || lens[u] == len_blk) vo[u] = __builtin_nontemporal_load(A + offs[u] + at);
        }
    }
#pragma unroll
    for (int u = 0; u < UU; ++u) {
        const int whole = lens[u] / NV * NV;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            const bool in = !RAGGED || own[j] < whole;
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const double x = (double)v[u][j][i];
                const double y = SUM ? acc[j][i] + x : combine(acc[j][i], x, op);
                acc[j][i] = in ? y : acc[j][i];
            }
        }
        if (odd_wave && (!RAGGED || lens[u] == len_blk)) odd = SUM ? odd + (double)vo[u] : combine(odd, (double)vo[u], op);
        if (RAGGED && lens[u] != len_blk && lens[u] != whole) {
            // the odd reals of a shorter tile lie in a whole slot of the block's tile: its owner reads them one by one
#pragma unroll
            for (int j = 0; j < J; ++j)
                if (own[j] == whole) {
#pragma unroll
                    for (int i = 0; i < NV - 1; ++i)
                        if (i < lens[u] - whole) acc[j][i] = combine(acc[j][i], (double)A[offs[u] + whole + i], op);
                }
        }
    }
}

// Kept coordinates of output q of a tile -> C offset in elements; false when q lies past the ragged edge.
template <bool CX>
__device__ __forceinline__ bool run_output(const RunArgs& a, int q, int x_here, int64_t& off) {
    off = 0;
    bool ok = true;
#pragma unroll
    for (int f = CX ? 1 : 0; f < RUN_AXES; ++f) {
        if (f < a.nf && !a.f_red[f]) {
            const int n = a.f_ext[f], h = q / n, c = q - h * n;
            q = h;
            off += (int64_t)c * a.f_so[f];
            if (f == a.nf - 1) ok = c < x_here;
        }
    }
    return ok;
}

template <class R, bool CX>
__device__ __forceinline__ void run_finish(const RunArgs& a, R* C, double re, double im) {
    if (CX) {
        double rr = a.alpha_re * re - a.alpha_im * im, ri = a.alpha_re * im + a.alpha_im * re;
        if (a.use_beta) {
            const double cr = C[0], ci = C[1];
            rr += a.beta_re * cr - a.beta_im * ci;
            ri += a.beta_re * ci + a.beta_im * cr;
        }
        C[0] = (R)rr;
        C[1] = (R)ri;
    } else {
        double r = a.alpha_re * re;
        if (a.use_beta) r += a.beta_re * (double)C[0];
        C[0] = (R)r;
    }
}

// Block b of a split -> origins in A (reals) and C (elements), and the indices of the ranged axis inside the tensor.
__device__ __forceinline__ void run_origin(const RunArgs& a, uint32_t bid, int64_t& org_in, int64_t& org_out, int& x_here) {
    org_in = org_out = 0;
    x_here = a.range;
    for (int g = 0; g < a.ng; ++g) {   // (the grid, and so every count, is below 2^31)
        const uint32_t n = (uint32_t)a.g_count[g], q = bid / n;
        const int64_t c = (int64_t)(bid - q * n);
        bid = q;
        org_in += c * a.g_si[g];
        org_out += c * a.g_so[g];
        if (g == 0 && a.g0_is_range) {
            const int64_t left = (int64_t)a.x_n - c * a.range;
            if (left < x_here) x_here = (int)left;
        }
    }
}

template <class R, bool CX, int J, bool SUM>
__global__ void __launch_bounds__(THREADS) reduce_run_kernel(RunArgs a) {
    prefetch_kernel_arguments<sizeof(RunArgs)>();
    constexpr int NV = 16 / sizeof(R);
    constexpr int NC = CX ? 2 : 1;
    constexpr int U = 8 / J;
    __shared__ double lds[RUN_REALS];
    const int tid = threadIdx.x;
    const int op = SUM ? (int)TFH_REDUCE_SUM : a.op;
    int64_t org_in, org_out;
    int x_here;
    run_origin(a, blockIdx.x, org_in, org_out, x_here);
    org_in = uniform64(org_in);
    const R* A = reinterpret_cast<const R*>(a.in) + org_in;
    // this block's tile: shorter than the others at the ragged edge of a kept ranged axis
    const int full = a.g0_is_range ? x_here * a.row_reals : a.tile_reals;
    const int whole = full / NV * NV, tail = full - whole;
    const int64_t it0 = (int64_t)blockIdx.y * a.per_split;
    const int64_t it1 = it0 + a.per_split < a.r_total ? it0 + a.per_split : a.r_total;
    RunOdometer odo;
    odo.off = 0;
    if (a.r_total < 0x7fffffff) {
        uint32_t lin = (uint32_t)it0;
#pragma unroll
        for (int r = 0; r < MAXR; ++r) {
            odo.c[r] = 0;
            if (r < a.nr) {
                const uint32_t n = (uint32_t)a.r_count[r], q = lin / n;
                odo.c[r] = lin - q * n;
                lin = q;
                odo.off += odo.c[r] * a.r_si[r];
            }
        }
    } else {
        int64_t lin = it0;
#pragma unroll
        for (int r = 0; r < MAXR; ++r) {
            odo.c[r] = 0;
            if (r < a.nr) {
                const int64_t q = lin / a.r_count[r];
                odo.c[r] = lin - q * a.r_count[r];
                lin = q;
                odo.off += odo.c[r] * a.r_si[r];
            }
        }
    }
    int own[J];   // first real of the thread's vector slots
#pragma unroll
    for (int j = 0; j < J; ++j) own[j] = (tid + THREADS * j) * NV;
    double acc[J][NV], odd = identity(op);
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[j][i] = identity(op);
    // a shorter tile among the reduced ones: the last index of r[0]
    const bool ragged_r = a.r0_is_range && (int64_t)a.x_n % a.range != 0;
    int64_t it = it0;
    for (; it + U <= it1; it += U) {
        if (ragged_r && odo.c[0] + U >= a.r_count[0]) run_tiles<R, J, U, SUM, true>(a, A, odo, own, full, op, acc, odd);
        else run_tiles<R, J, U, SUM, false>(a, A, odo, own, full, op, acc, odd);
    }
    for (; it < it1; ++it) {
        if (ragged_r) run_tiles<R, J, 1, SUM, true>(a, A, odo, own, full, op, acc, odd);
        else run_tiles<R, J, 1, SUM, false>(a, A, odo, own, full, op, acc, odd);
    }
    // accumulators -> LDS in tile order
#pragma unroll
    for (int j = 0; j < J; ++j) {
        if (own[j] < whole) {
#pragma unroll
            for (int i = 0; i < NV; ++i) lds[own[j] + i] = acc[j][i];
        }
    }
    if (tid < tail) lds[whole + tid] = odd;
    // (positions from the block's tile length to the full tile's hold nothing: they are coordinates past the ragged
    // edge of a kept axis, folded into outputs that are not written)
    __syncthreads();
    // fold the reduced tile axes, innermost first; a folded axis keeps extent 1
    int ext[RUN_AXES];
#pragma unroll
    for (int f = 0; f < RUN_AXES; ++f) ext[f] = f < a.nf ? a.f_ext[f] : 1;
#pragma unroll
    for (int f = 0; f < RUN_AXES; ++f) {
        if (f >= a.nf || !a.f_red[f]) continue;
        int inner = 1, outer = 1;
#pragma unroll
        for (int k = 0; k < RUN_AXES; ++k) {
            if (k < f) inner *= ext[k];
            if (k > f) outer *= ext[k];
        }
        const int count = inner * outer;
        int n = ext[f];
        while (n > 1) {
            int groups = THREADS / count;
            if (groups > (n + 15) / 16) groups = (n + 15) / 16;
            if (groups < 1) groups = 1;
            const int each = (n + groups - 1) / groups;
            groups = (n + each - 1) / each;
            const int total = count * groups;   // at most RUN_REALS
            double s[RUN_REALS / THREADS];
#pragma unroll
            for (int k = 0; k < RUN_REALS / THREADS; ++k) {
                const int o = tid + THREADS * k;
                s[k] = identity(op);
                if (o < total) {
                    const int in = o % inner, rest = o / inner, g = rest % groups, ou = rest / groups;
                    const int k0 = g * each, k1 = k0 + each < n ? k0 + each : n;
                    const double* p = lds + ((int64_t)ou * n + k0) * inner + in;
                    for (int x = k0; x < k1; ++x, p += inner) s[k] = combine(s[k], *p, op);
                }
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < RUN_REALS / THREADS; ++k) {
                const int o = tid + THREADS * k;
                if (o < total) lds[o] = s[k];
            }
            __syncthreads();
            n = groups;
        }
        ext[f] = 1;
    }
    // the tile's outputs
    const int nq = a.kept_per_tile;
    for (int q = tid; q < nq; q += THREADS) {
        int64_t off;
        if (!run_output<CX>(a, q, x_here, off)) continue;
        const double re = lds[q * NC], im = CX ? lds[q * NC + 1] : 0.0;
        if (a.nsplit > 1) {
            double* P = a.partial + (((int64_t)blockIdx.y * a.blocks + blockIdx.x) * nq + q) * NC;
            P[0] = re;
            if (CX) P[1] = im;
        } else {
            run_finish<R, CX>(a, reinterpret_cast<R*>(a.out) + (org_out + off) * NC, re, im);
        }
    }
}

// Every tile axis reduced (rows summed whole, a full reduction): a tile has no coordinates worth keeping, so a thread
// adds everything it reads into one accumulator, and a block takes KS outputs that are neighbours along the kept axes
// outside the tile, in step, so that rows of a few KB still give every thread eight loads in flight and one
// exchange through LDS serves KS outputs.
template <class R, bool CX, int J, int KS, bool SUM>
__global__ void __launch_bounds__(THREADS) reduce_run_rows_kernel(RunArgs a) {
    prefetch_kernel_arguments<sizeof(RunArgs)>();
    constexpr int NV = 16 / sizeof(R);
    constexpr int NC = CX ? 2 : 1;
    constexpr int U = J * KS >= 8 ? 1 : 8 / (J * KS);
    typedef typename RunVec<R, NV>::type V;
    __shared__ double lds[KS * 4 * 2];
    const int tid = threadIdx.x;
    const int op = SUM ? (int)TFH_REDUCE_SUM : a.op;
    const uint32_t item0 = blockIdx.x * KS, items = (uint32_t)a.blocks;
    int64_t org[KS];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
        int64_t org_out;
        int x_here;
        run_origin(a, item0 + k < items ? item0 + k : items - 1, org[k], org_out, x_here);
        org[k] = uniform64(org[k]);
    }
    const R* A = reinterpret_cast<const R*>(a.in);
    const int full = a.tile_reals;
    const int64_t it0 = (int64_t)blockIdx.y * a.per_split;
    const int64_t it1 = it0 + a.per_split < a.r_total ? it0 + a.per_split : a.r_total;
    RunOdometer odo;
    odo.off = 0;
    {
        int64_t lin = it0;
#pragma unroll
        for (int r = 0; r < MAXR; ++r) {
            odo.c[r] = 0;
            if (r < a.nr) {
                const int64_t q = lin / a.r_count[r];
                odo.c[r] = lin - q * a.r_count[r];
                lin = q;
                odo.off += odo.c[r] * a.r_si[r];
            }
        }
    }
    int own[J];
#pragma unroll
    for (int j = 0; j < J; ++j) own[j] = (tid + THREADS * j) * NV;
    double re[KS], im[KS];
#pragma unroll
    for (int k = 0; k < KS; ++k) {
        re[k] = identity(op);
        im[k] = 0.0;
    }
    const bool ragged_r = a.r0_is_range && (int64_t)a.x_n % a.range != 0;
    for (int64_t it = it0; it < it1; it += U) {
        int64_t offs[U];
        int lens[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            offs[u] = uniform64(odo.off);
            lens[u] = full;
            if (ragged_r) {
                const int64_t left = (int64_t)a.x_n - odo.c[0] * a.range;
                lens[u] = (int)(left < a.range ? left : a.range) * a.row_reals;
            }
            if (it + u >= it1) lens[u] = 0;
            else run_advance(a, odo);
        }
        V v[U][KS][J];
        R vo[U][KS];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int last = lens[u] / NV - 1, whole = (last + 1) * NV, rest = lens[u] - whole;
#pragma unroll
            for (int k = 0; k < KS; ++k) {
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const int at = own[j] < last * NV ? own[j] : last * NV;
                    v[u][k][j] = V{};
                    if (last >= 0) v[u][k][j] = __builtin_nontemporal_load(reinterpret_cast<const V*>(A + org[k] + offs[u] + at));
                }
                vo[u][k] = R(0);
                if (rest > 0 && tid < 64) vo[u][k] = __builtin_nontemporal_load(A + org[k] + offs[u] + whole + (tid < rest ? tid : rest - 1));
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int whole = lens[u] / NV * NV, rest = lens[u] - whole;
#pragma unroll
            for (int k = 0; k < KS; ++k) {
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const bool in = own[j] < whole;
#pragma unroll
                    for (int i = 0; i < NV; ++i) {
                        const double x = (double)v[u][k][j][i];
                        if (CX && (i & 1)) {
                            im[k] = in ? im[k] + x : im[k];
                        } else {
                            const double y = SUM ? re[k] + x : combine(re[k], x, op);
                            re[k] = in ? y : re[k];
                        }
                    }
                }
                if (tid < rest) {
                    const double x = (double)vo[u][k];
                    if (CX && (tid & 1)) im[k] += x;
                    else re[k] = combine(re[k], x, op);
                }
            }
        }
    }
#pragma unroll
    for (int k = 0; k < KS; ++k) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            re[k] = combine(re[k], __shfl_xor(re[k], d), op);
            if (CX) im[k] += __shfl_xor(im[k], d);
        }
        if ((tid & 63) == 0) {
            lds[(k * 4 + (tid >> 6)) * 2] = re[k];
            lds[(k * 4 + (tid >> 6)) * 2 + 1] = im[k];
        }
    }
    __syncthreads();
    if (tid >= KS || item0 + tid >= items) return;
    const double* w = lds + tid * 8;
    const double sre = combine(combine(w[0], w[2], op), combine(w[4], w[6], op), op), sim = (w[1] + w[3]) + (w[5] + w[7]);
    if (a.nsplit > 1) {
        double* P = a.partial + ((int64_t)blockIdx.y * a.blocks + item0 + tid) * NC;
        P[0] = sre;
        if (CX) P[1] = sim;
    } else {
        int64_t org_in, org_out;
        int x_here;
        run_origin(a, item0 + tid, org_in, org_out, x_here);
        run_finish<R, CX>(a, reinterpret_cast<R*>(a.out) + org_out * NC, sre, sim);
    }
}

// Second pass of a split walk: `team` threads (a power of two) per output add the partial results split, split +
// team, ... and meet in an LDS tree.
template <class R, bool CX>
__global__ void __launch_bounds__(THREADS) reduce_run_fold_kernel(RunArgs a, int team) {
    constexpr int NC = CX ? 2 : 1;
    __shared__ double lds[THREADS * NC];
    const int tid = threadIdx.x, per = THREADS / team, g = tid / per;
    const int64_t outputs = a.blocks * a.kept_per_tile;
    const int64_t o = (int64_t)blockIdx.x * per + tid % per;
    const int op = a.op;
    double re = identity(op), im = 0.0;
    if (o < outputs) {
        // eight partial results in flight at a time (each is a trip to memory), added in the order of the splits
        for (int s0 = g; s0 < a.nsplit; s0 += 8 * team) {
            double pr[8], pi[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int s = s0 + i * team;
                pr[i] = identity(op);
                pi[i] = 0.0;
                if (s < a.nsplit) {
                    const double* P = a.partial + ((int64_t)s * outputs + o) * NC;
                    pr[i] = P[0];
                    if (CX) pi[i] = P[1];
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                re = combine(re, pr[i], op);
                if (CX) im += pi[i];
            }
        }
    }
    if (team > 1) {
        lds[tid * NC] = re;
        if (CX) lds[tid * NC + 1] = im;
        __syncthreads();
        for (int stride = THREADS / 2; stride >= per; stride >>= 1) {
            if (tid < stride) {
                lds[tid * NC] = combine(lds[tid * NC], lds[(tid + stride) * NC], op);
                if (CX) lds[tid * NC + 1] += lds[(tid + stride) * NC + 1];
            }
            __syncthreads();
        }
        re = lds[tid * NC];
        if (CX) im = lds[tid * NC + 1];
    }
    if (g != 0 || o >= outputs) return;
    const int64_t b = o / a.kept_per_tile;
    const int q = (int)(o - b * a.kept_per_tile);
    int64_t org_in, org_out, off;
    int x_here;
    run_origin(a, (uint32_t)b, org_in, org_out, x_here);
    if (!run_output<CX>(a, q, x_here, off)) return;
    run_finish<R, CX>(a, reinterpret_cast<R*>(a.out) + (org_out + off) * NC, re, im);
}

template <class R, bool CX, int J>
void launch_run_j(const RunArgs& ra, dim3 grid, hipStream_t st) {
    if (ra.op == TFH_REDUCE_SUM) TFH_LAUNCH_TIMED((reduce_run_kernel<R, CX, J, true>), grid, dim3(THREADS), 0, st, ra);
    else TFH_LAUNCH_TIMED((reduce_run_kernel<R, CX, J, false>), grid, dim3(THREADS), 0, st, ra);
}
template <class R, bool CX>
void launch_run(const RunArgs& ra, int j, dim3 grid, hipStream_t st) {
    if (j == 1) launch_run_j<R, CX, 1>(ra, grid, st);
    else if (j == 2) launch_run_j<R, CX, 2>(ra, grid, st);
    else if constexpr (sizeof(R) == 8) launch_run_j<R, CX, 4>(ra, grid, st);
}
template <class R, bool CX, int J, int KS>
void launch_rows_jk(const RunArgs& ra, dim3 grid, hipStream_t st) {
    if (ra.op == TFH_REDUCE_SUM) TFH_LAUNCH_TIMED((reduce_run_rows_kernel<R, CX, J, KS, true>), grid, dim3(THREADS), 0, st, ra);
    else TFH_LAUNCH_TIMED((reduce_run_rows_kernel<R, CX, J, KS, false>), grid, dim3(THREADS), 0, st, ra);
}
template <class R, bool CX>
void launch_rows(const RunArgs& ra, int j, int ks, dim3 grid, hipStream_t st) {
    if (j == 1) {
        if (ks == 8) launch_rows_jk<R, CX, 1, 8>(ra, grid, st);
        else if (ks == 4) launch_rows_jk<R, CX, 1, 4>(ra, grid, st);
        else if (ks == 2) launch_rows_jk<R, CX, 1, 2>(ra, grid, st);
        else launch_rows_jk<R, CX, 1, 1>(ra, grid, st);
    } else if (j == 2) {
        if (ks == 4) launch_rows_jk<R, CX, 2, 4>(ra, grid, st);
        else if (ks == 2) launch_rows_jk<R, CX, 2, 2>(ra, grid, st);
        else launch_rows_jk<R, CX, 2, 1>(ra, grid, st);
    } else if constexpr (sizeof(R) == 8) {
        if (ks == 2) launch_rows_jk<R, CX, 4, 2>(ra, grid, st);
        else launch_rows_jk<R, CX, 4, 1>(ra, grid, st);
    }
}
}  // namespace

namespace {
// Returns true when the dense-run kernel was launched.
bool try_run_reduce(int dtype, const void* a, void* c, const std::vector<Axis>& kept, const std::vector<Axis>& red, int reduce_op,
                    Scalar alpha, Scalar beta, void* stream, int32_t& status) {
    status = TFH_OK;
    const bool cx = is_complex(dtype), dbl = is_double(dtype);
    const int nc = cx ? 2 : 1, nv = dbl ? 2 : 4;
    if (cx && reduce_op != TFH_REDUCE_SUM) return false;
    struct Ax {
        int64_t n, si, so;
        bool red;
    };
    std::vector<Ax> all;
    int64_t total = 1;
    for (auto& x : kept) {
        if (x.n == 1) continue;
        if (x.s[0] <= 0 || x.s[1] == 0) return false;
        all.push_back({x.n, x.s[0], x.s[1], false});
        total *= x.n;
    }
    for (auto& x : red) {
        if (x.n == 1) continue;
        if (x.s[0] <= 0) return false;
        all.push_back({x.n, x.s[0], 0, true});
        total *= x.n;
    }
    if (total < 65536) return false;
    std::stable_sort(all.begin(), all.end(), [](const Ax& x, const Ax& y) { return x.si < y.si; });
    // neighbours of one kind that are dense in A (and in C, when kept) are one axis
    std::vector<Ax> ax;
    for (auto& x : all) {
        if (!ax.empty() && ax.back().red == x.red && x.si == ax.back().si * ax.back().n &&
            (x.red || x.so == ax.back().so * ax.back().n)) {
            ax.back().n *= x.n;
        } else {
            ax.push_back(x);
        }
    }
    // the dense prefix, and a tile in it
    size_t np = 0;
    for (int64_t run = 1; np < ax.size() && ax[np].si == run; ++np) run *= ax[np].n;
    if (np == 0) return false;
    RunArgs ra;
    std::memset(&ra, 0, sizeof ra);
    if (cx) {
        ra.f_ext[0] = 2;
        ra.nf = 1;
    }
    auto plan_tile = [&](int64_t cap, size_t& whole, int64_t& range) {   // axes [0, whole) whole, `range` indices of axis `whole`
        int64_t w = nc;
        whole = 0;
        range = 0;
        while (whole < np && (int)whole + (cx ? 1 : 0) < RUN_AXES - 1 && w * ax[whole].n <= cap) w *= ax[whole++].n;
        if (whole < np && w <= cap) {
            const int64_t t0 = std::max<int64_t>(1, cap / w), pieces = (ax[whole].n + t0 - 1) / t0;
            if (t0 >= 2 || whole == 0) range = (ax[whole].n + pieces - 1) / pieces;   // (one index per tile: an axis outside the tile)
        }
        return w * std::max<int64_t>(1, range);
    };
    // The tile: as large as the vector slots of a block hold, unless that leaves the chip short of blocks.  Blocks come
    // from the kept axes outside the tile and from splitting the walk, which is bounded by the size of the partial
    // results (a share of A's) -- so with few outputs per tile a smaller tile is what gives more blocks.
    constexpr int64_t target = 1280;   // blocks of a split walk: five per CU, all resident at once
    constexpr int64_t minper = 2;      // tiles per block at least
    struct Choice {
        size_t whole;
        int64_t range, tile_reals, kept_blocks, nsplit;
    };
    auto evaluate = [&](int64_t cap) {
        Choice ch;
        ch.tile_reals = plan_tile(cap, ch.whole, ch.range);
        ch.kept_blocks = 1;
        int64_t walk = 1, kept_in_tile = 1;
        for (size_t i = 0; i < ax.size(); ++i) {
            const bool ranged = i == ch.whole && ch.range > 0;
            const int64_t outside = i < ch.whole ? 1 : (ranged ? (ax[i].n + ch.range - 1) / ch.range : ax[i].n);
            const int64_t inside = i < ch.whole ? ax[i].n : (ranged ? ch.range : 1);
            if (ax[i].red) walk *= outside;
            else ch.kept_blocks *= outside, kept_in_tile *= inside;
        }
        ch.nsplit = 1;
        // (a walk of three batches of loads or fewer on 64 blocks or more stays one launch: the second launch of a
        // split walk costs 4-5 us, as much as those batches)
        const bool short_walk = ch.kept_blocks >= 64 && walk * ch.tile_reals * (dbl ? 8 : 4) <= 98304;
        if (ch.kept_blocks < 768 && walk >= 2 * minper && !short_walk) {
            const int64_t outputs = ch.kept_blocks * kept_in_tile;
            ch.nsplit = std::min<int64_t>(target / ch.kept_blocks, walk / minper);
            ch.nsplit = std::min<int64_t>(ch.nsplit, std::max<int64_t>(1, total / (outputs * 48)));
            ch.nsplit = std::max<int64_t>(1, std::min<int64_t>(ch.nsplit, 65535));
        }
        return ch;
    };
    Choice best = evaluate(RUN_REALS);
    for (int64_t cap = RUN_REALS / 2; cap >= (int64_t)THREADS * nv && best.kept_blocks * best.nsplit < 1024; cap >>= 1) {
        const Choice ch = evaluate(cap);
        if (ch.kept_blocks * ch.nsplit > best.kept_blocks * best.nsplit) best = ch;
    }
    size_t whole = best.whole;
    int64_t range = best.range;
    const int64_t tile_reals = best.tile_reals;
    if (tile_reals < 256) return false;   // a short dense prefix: most lanes would idle
    int j = dbl ? 4 : 2;
    while (j > 1 && (tile_reals + nv - 1) / nv <= (int64_t)THREADS * (j / 2)) j >>= 1;
    // tile axes
    int64_t kept_per_tile = 1;
    for (size_t i = 0; i < whole + (range ? 1 : 0); ++i) {
        const int f = ra.nf++;
        const int64_t e = (i == whole) ? range : ax[i].n;
        ra.f_ext[f] = (int32_t)e;
        ra.f_red[f] = ax[i].red;
        ra.f_so[f] = ax[i].so;
        if (!ax[i].red) kept_per_tile *= e;
    }
    if (!range) {   // the tile is the whole prefix: its outermost axis is the ranged one, with a single range
        if (whole == 0) return false;
        range = ax[whole - 1].n;
        --whole;
    }
    ra.tile_reals = (int32_t)tile_reals;
    ra.range = (int32_t)range;
    ra.x_n = (int32_t)ax[whole].n;
    if (ax[whole].n > 0x7fffffff) {
        // (the extent of the ranged axis is kept in 32 bits)
        return false;
    }
    ra.row_reals = (int32_t)(tile_reals / range);
    ra.kept_per_tile = (int32_t)kept_per_tile;
    ra.all_reduced = 1;
    for (int f = cx ? 1 : 0; f < ra.nf; ++f) ra.all_reduced &= ra.f_red[f];
    const int64_t pieces = (ax[whole].n + range - 1) / range;
    int64_t blocks = 1;
    ra.r_total = 1;
    if (pieces > 1) {
        if (ax[whole].red) {
            ra.r0_is_range = 1;
            ra.r_count[0] = pieces;
            ra.r_si[0] = ax[whole].si * range * nc;
            ra.nr = 1;
            ra.r_total = pieces;
        } else {
            ra.g0_is_range = 1;
            ra.g_count[0] = pieces;
            ra.g_si[0] = ax[whole].si * range * nc;
            ra.g_so[0] = ax[whole].so * range;
            ra.ng = 1;
            blocks = pieces;
        }
    }
    for (size_t i = whole + 1; i < ax.size(); ++i) {
        if (ax[i].red) {
            if (ra.nr == MAXR) return false;
            ra.r_count[ra.nr] = ax[i].n;
            ra.r_si[ra.nr] = ax[i].si * nc;
            ++ra.nr;
            ra.r_total *= ax[i].n;
        } else {
            if (ra.ng == MAXG) return false;
            ra.g_count[ra.ng] = ax[i].n;
            ra.g_si[ra.ng] = ax[i].si * nc;
            ra.g_so[ra.ng] = ax[i].so;
            ++ra.ng;
            blocks *= ax[i].n;
            if (blocks > 0x7fffffffll) return false;
        }
    }
    if (ra.nr == 0) {
        ra.nr = 1;
        ra.r_count[0] = 1;
    }
    ra.blocks = blocks;
    int64_t nsplit = best.nsplit;
    ra.per_split = (ra.r_total + nsplit - 1) / nsplit;
    nsplit = (ra.r_total + ra.per_split - 1) / ra.per_split;
    ra.nsplit = (int32_t)nsplit;
    ra.in = a;
    ra.out = c;
    ra.op = reduce_op;
    ra.alpha_re = alpha.re;
    ra.alpha_im = alpha.im;
    ra.beta_re = beta.re;
    ra.beta_im = beta.im;
    ra.use_beta = !beta.is_zero();
    if (nsplit > 1) {
        void* ws = nullptr;
        const size_t bytes = (size_t)nsplit * (size_t)blocks * (size_t)kept_per_tile * nc * sizeof(double);
        if ((status = workspace(stream, bytes, &ws)) != TFH_OK) return true;
        ra.partial = (double*)ws;
    }
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_REDUCE, stream);
    if (ra.all_reduced) {
        // several outputs per block when each has a short walk
        int ks = 8 / j;
        while (ks > 1 && ((int64_t)ks * ra.per_split > 16 || blocks / ks < 1024)) ks >>= 1;
        const dim3 grid((uint32_t)((blocks + ks - 1) / ks), (uint32_t)nsplit, 1);
        switch (dtype) {
            case TFH_F32: launch_rows<float, false>(ra, j, ks, grid, st); break;
            case TFH_F64: launch_rows<double, false>(ra, j, ks, grid, st); break;
            case TFH_C64: launch_rows<float, true>(ra, j, ks, grid, st); break;
            default: launch_rows<double, true>(ra, j, ks, grid, st); break;
        }
    } else {
        const dim3 grid((uint32_t)blocks, (uint32_t)nsplit, 1);
        switch (dtype) {
            case TFH_F32: launch_run<float, false>(ra, j, grid, st); break;
            case TFH_F64: launch_run<double, false>(ra, j, grid, st); break;
            case TFH_C64: launch_run<float, true>(ra, j, grid, st); break;
            default: launch_run<double, true>(ra, j, grid, st); break;
        }
    }
    prof_end(prof, stream);
    if ((status = hip_check(hipGetLastError(), "reduce kernel launch")) != TFH_OK) return true;
    if (nsplit > 1) {
        const int64_t outputs = blocks * kept_per_tile;
        int team = 1;
        while (team < THREADS && team * 2 <= nsplit && outputs * team < 65536) team *= 2;
        const int per = THREADS / team;
        const dim3 g2((uint32_t)((outputs + per - 1) / per));
        switch (dtype) {
            case TFH_F32: hipLaunchKernelGGL((reduce_run_fold_kernel<float, false>), g2, dim3(THREADS), 0, st, ra, team); break;
            case TFH_F64: hipLaunchKernelGGL((reduce_run_fold_kernel<double, false>), g2, dim3(THREADS), 0, st, ra, team); break;
            case TFH_C64: hipLaunchKernelGGL((reduce_run_fold_kernel<float, true>), g2, dim3(THREADS), 0, st, ra, team); break;
            default: hipLaunchKernelGGL((reduce_run_fold_kernel<double, true>), g2, dim3(THREADS), 0, st, ra, team); break;
        }
        status = hip_check(hipGetLastError(), "reduce fold launch");
    }
    return true;
}
}  // namespace

int32_t launch_reduce(int dtype, const void* a, void* c, std::vector<Axis> kept, std::vector<Axis> red, int reduce_op,
                      Scalar alpha, Scalar beta, void* stream) {
    const int rb = is_double(dtype) ? 8 : 4;
    if (((uintptr_t)a % rb) || ((uintptr_t)c % rb)) return set_error(TFH_ERR_STRIDED, "view base is not aligned");
    for (auto& x : kept)
        if (x.n == 0) return TFH_OK;  // no outputs
    int64_t nred = 1;
    for (auto& x : red) nred *= x.n;
    if (nred == 0) {
        // empty reduction: every output is alpha*identity + beta*C; sum -> 0
        if (reduce_op != TFH_REDUCE_SUM) return set_error(TFH_ERR_INVALID_ARGUMENT, "max/min over an empty extent");
        red.clear();
        // scale C by beta through the copy kernel (in = out, alpha = 0 is not safe for NaN; use fill when beta == 0)
        std::vector<Axis> ax;
        for (auto& x : kept) ax.push_back(Axis{x.n, {x.s[1], x.s[1], 0}, x.label});
        if (beta.is_zero()) return launch_fill(dtype, c, ax, Scalar{0, 0}, stream);
        return launch_copy(dtype, c, c, ax, beta, Scalar{0, 0}, false, stream);
    }
    {
        int32_t st_fast = TFH_OK;
        if (try_fast_reduce(dtype, a, c, kept, red, reduce_op, alpha, beta, stream, st_fast)) return st_fast;
        if (try_shortrow_reduce(dtype, a, c, kept, red, reduce_op, alpha, beta, stream, st_fast)) return st_fast;
        if (try_run_reduce(dtype, a, c, kept, red, reduce_op, alpha, beta, stream, st_fast)) return st_fast;
    }
    for (auto& x : kept) x.s[2] = 0;
    for (auto& x : red) x.s[1] = x.s[2] = 0;
    return launch_reduce_general(dtype, a, nullptr, c, kept, red, reduce_op, alpha, beta, stream);
}

// The general kernel for any extents and strides.  Axis slots: 0 = A, 1 = C, 2 = B (the second operand of a product
// reduction, b != nullptr; zero strides otherwise).
int32_t launch_reduce_general(int dtype, const void* a, const void* b, void* c, std::vector<Axis> kept, std::vector<Axis> red,
                              int reduce_op, Scalar alpha, Scalar beta, void* stream) {
    // merge axes (kept and reduced separately)
    std::stable_sort(kept.begin(), kept.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    fuse_axes(kept, 3);
    auto key_red = [](const Axis& x) { return x.s[0] == 0 ? INT64_MAX : std::llabs(x.s[0]); };
    std::stable_sort(red.begin(), red.end(), [&](const Axis& x, const Axis& y) { return key_red(x) > key_red(y); });
    fuse_axes(red, 3);
    for (auto& x : kept)
        if (x.s[1] == 0) return set_error(TFH_ERR_STRIDED, "output view has stride 0 on an axis of extent %lld", (long long)x.n);
    struct Ax {
        Axis a;
        bool red;
        int tl;  // log2 tile extent
    };
    std::vector<Ax> all;
    for (auto& x : kept) all.push_back({x, false, 0});
    for (auto& x : red) all.push_back({x, true, 0});
    if ((int)all.size() > MAXG) return set_error(TFH_ERR_INVALID_ARGUMENT, "more than %d non-mergeable axes", MAXG);
    auto key = [](const Ax& x) { return x.a.s[0] == 0 ? INT64_MAX : std::llabs(x.a.s[0]); };
    std::stable_sort(all.begin(), all.end(), [&](const Ax& x, const Ax& y) { return key(x) < key(y); });
    ReduceArgs ra;
    std::memset(&ra, 0, sizeof ra);
    int bits = 8, nt = 0;
    for (auto& x : all) {
        if (bits == 0 || nt == MAXT) break;
        int t = std::min(ceil_log2(x.a.n), bits);
        if (x.red && x.a.n >= 64) {
            // leave a thread at least eight serial steps along a reduced axis: a short row spread over all 256 lanes
            // would be one load per thread and a full fold per row (rows of 300 f64: 0.6 TB/s).  Extents below 64
            // keep their lanes (as serial axes they would count against the limit on serial reduced axes).
            int cap = 0;
            while (((int64_t)16 << cap) <= x.a.n) ++cap;
            t = std::min(t, cap);
        }
        if (t == 0) continue;
        x.tl = t;
        bits -= t;
        ++nt;
    }
    int shift = 0;
    ra.nt = 0;
    std::vector<int> tid_of(all.size(), -1);
    for (size_t i = 0; i < all.size(); ++i) {
        if (all[i].tl == 0) continue;
        int t = ra.nt++;
        tid_of[i] = t;
        ra.t_shift[t] = shift;
        ra.t_mask[t] = (1 << all[i].tl) - 1;
        ra.t_red[t] = all[i].red;
        ra.t_sa[t] = all[i].a.s[0];
        ra.t_sc[t] = all[i].a.s[1];
        ra.t_sb[t] = all[i].a.s[2];
        ra.t_n[t] = all[i].a.n;
        if (all[i].red) ra.red_bits |= ra.t_mask[t] << shift;
        shift += all[i].tl;
    }
    ra.tile_elems = 1 << shift;
    // kept outer axes -> grid.x ; reduced outer axes -> serial loop
    uint64_t blocks = 1;
    ra.r_total = 1;
    for (int r = 0; r < MAXR; ++r) {
        ra.r_count[r] = 1;
        ra.r_n[r] = 1;
        ra.r_text[r] = 1;
        ra.r_tid[r] = -1;
    }
    for (size_t i = 0; i < all.size(); ++i) {
        int64_t text = (int64_t)1 << all[i].tl;
        int64_t cnt = (all[i].a.n + text - 1) / text;
        if (cnt <= 1) continue;
        if (all[i].red) {
            if (ra.nr == MAXR) return set_error(TFH_ERR_INVALID_ARGUMENT, "more than %d non-mergeable reduced axes outside the thread tile", MAXR);
            int r = ra.nr++;
            ra.r_count[r] = cnt;
            ra.r_sa[r] = all[i].a.s[0] * text;
            ra.r_sb[r] = all[i].a.s[2] * text;
            ra.r_n[r] = all[i].a.n;
            ra.r_tid[r] = tid_of[i];
            ra.r_text[r] = (int32_t)text;
            ra.r_total *= cnt;
        } else {
            int g = ra.ng++;
            ra.g_count[g] = cnt;
            ra.g_sa[g] = all[i].a.s[0] * text;
            ra.g_sc[g] = all[i].a.s[1] * text;
            ra.g_sb[g] = all[i].a.s[2] * text;
            ra.g_tid[g] = tid_of[i];
            ra.g_text[g] = (int32_t)text;
            blocks *= (uint64_t)cnt;
        }
    }
    if (ra.nr == 0) ra.nr = 1;  // a single pass through the loop
    if (blocks > 0x7fffffffull) return set_error(TFH_ERR_INVALID_ARGUMENT, "tensor too large for one launch");
    // split a long serial range when there are too few blocks to fill 256 CUs
    int nchunks = 1;
    if (blocks < 1024 && ra.r_total >= 64) {
        nchunks = (int)std::min<int64_t>((2048 + (int64_t)blocks - 1) / (int64_t)blocks, ra.r_total / 16);
        nchunks = std::max(1, std::min(nchunks, 65535));
    }
    ra.nchunks = nchunks;
    ra.kept_slots = (int64_t)blocks * THREADS;
    ra.in = a;
    ra.in_b = b;
    ra.out = c;
    ra.op = reduce_op;
    ra.alpha_re = alpha.re;
    ra.alpha_im = alpha.im;
    ra.beta_re = beta.re;
    ra.beta_im = beta.im;
    ra.use_beta = !beta.is_zero();
    const bool cx = is_complex(dtype);
    if (nchunks > 1) {
        void* ws = nullptr;
        size_t bytes = (size_t)nchunks * (size_t)ra.kept_slots * (cx ? 2 : 1) * sizeof(double);
        if (int32_t e = workspace(stream, bytes, &ws)) return e;
        ra.partial = (double*)ws;
    }
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((uint32_t)blocks, (uint32_t)nchunks, 1), block(THREADS);
    const int prof = prof_begin(b ? PROF_CONTRACT : PROF_REDUCE, stream);
    if (b) {
        switch (dtype) {
            case TFH_F32: TFH_LAUNCH_TIMED((reduce_kernel<float, false, true>), grid, block, 0, st, ra); break;
            case TFH_F64: TFH_LAUNCH_TIMED((reduce_kernel<double, false, true>), grid, block, 0, st, ra); break;
            case TFH_C64: TFH_LAUNCH_TIMED((reduce_kernel<float, true, true>), grid, block, 0, st, ra); break;
            default: TFH_LAUNCH_TIMED((reduce_kernel<double, true, true>), grid, block, 0, st, ra); break;
        }
    } else {
        switch (dtype) {
            case TFH_F32: TFH_LAUNCH_TIMED((reduce_kernel<float, false>), grid, block, 0, st, ra); break;
            case TFH_F64: TFH_LAUNCH_TIMED((reduce_kernel<double, false>), grid, block, 0, st, ra); break;
            case TFH_C64: TFH_LAUNCH_TIMED((reduce_kernel<float, true>), grid, block, 0, st, ra); break;
            default: TFH_LAUNCH_TIMED((reduce_kernel<double, true>), grid, block, 0, st, ra); break;
        }
    }
    prof_end(prof, stream);
    if (int32_t e = hip_check(hipGetLastError(), "reduce kernel launch")) return e;
    if (nchunks > 1) {
        dim3 g2((uint32_t)blocks, 1, 1);
        switch (dtype) {
            case TFH_F32: hipLaunchKernelGGL((reduce_finalize_kernel<float, false>), g2, block, 0, st, ra); break;
            case TFH_F64: hipLaunchKernelGGL((reduce_finalize_kernel<double, false>), g2, block, 0, st, ra); break;
            case TFH_C64: hipLaunchKernelGGL((reduce_finalize_kernel<float, true>), g2, block, 0, st, ra); break;
            default: hipLaunchKernelGGL((reduce_finalize_kernel<double, true>), g2, block, 0, st, ra); break;
        }
        if (int32_t e = hip_check(hipGetLastError(), "reduce finalize launch")) return e;
    }
    return TFH_OK;
}

}  // namespace tfh
