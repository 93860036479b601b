// k_dot.hip -- contractions with (almost) no output per reduced element: matrix-vector and vector-matrix products,
// dot products and batched dot products -- PrimDescriptor::Contract (tenferro-prims/src/lib.rs:227-239) when one
// free group is empty or tiny.  C[kept] = alpha * sum_red A[kept, red] * B[kept, red] + beta * C, where either operand
// may lack (stride 0) any kept axis.
//
// A tiled MFMA kernel computes a 64x64 tile for one useful column there and is bound by the latency of its small loads
// (an 8192 x 8192 f64 matrix times a vector: 2.3 TB/s).  These products are reductions of an elementwise product and
// take the layout of the fast reduction kernel instead: the 256 threads of a block tile the axes that are fastest
// in the memory of A (the larger operand), kept or reduced alike, with 16-byte loads along its contiguous axis; B is
// read at the same coordinates through its own strides (a vector load when it is contiguous along that axis too, one
// element broadcast over the lanes' vector when it has stride 0 there); a thread walks the remaining reduced range
// serially with a rolling window of loads, lanes that share an output fold with lane exchanges and LDS, and with few
// outputs the serial range is split over blockIdx.y into raw partials that a second launch folds in a fixed order.
// Products and sums are in f64 for every dtype.  HBM-bound: algorithmic bytes = sizeof(A) + sizeof(B) + sizeof(C).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "internal.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

constexpr int MAXT = 4, MAXG = 16, MAXR = 4, THREADS = 256;
constexpr int MAX_RTAB = 1024;

struct DotArgs {
    const void* a;
    const void* b;
    void* c;
    int32_t nt, ng, nr;
    int32_t red_bits, use_beta;
    int32_t t_shift[MAXT], t_mask[MAXT], t_red[MAXT];
    int64_t t_sa[MAXT], t_sb[MAXT], t_sc[MAXT];
    int64_t g_count[MAXG], g_sa[MAXG], g_sb[MAXG], g_sc[MAXG];
    int64_t r_count[MAXR], r_sa[MAXR], r_sb[MAXR];
    int32_t r_total;
    int32_t rot_shift;   // as in the reduction kernel: >= 0 rotates the serial start by block group (mode 0), < 0 off
    int32_t mode, nchunks, rps, nblocks;   // as in the reduction kernel: 0 whole range, 1 write partials, 2 fold partials
    double* partial;                        // [nchunks][nblocks][THREADS][NV]
    int64_t vc_stride;                      // C stride between the VEC outputs of one lane (contiguous axis kept)
    double alpha_re, alpha_im, beta_re, beta_im;
};

template <class R, int N>
struct alignas(sizeof(R) * N) RVec {
    R v[N];
};
template <class R, int N> struct RawV { typedef R type __attribute__((ext_vector_type(N))); };
template <class R> struct RawV<R, 1> { typedef R type; };
template <class R, int N>
__device__ __forceinline__ RVec<R, N> load_stream(const R* p) {
    typedef typename RawV<R, N>::type Raw;
    return __builtin_bit_cast(RVec<R, N>, __builtin_nontemporal_load(reinterpret_cast<const Raw*>(p)));
}

// R: component type.  VEC: elements of A per load (real) -- a complex element is one load of its two components.
// KV: A's contiguous axis is kept (VEC outputs per lane).  BB: B has stride 0 along that axis.  CX: complex product.
template <class R, int VEC, bool KV, bool BB, bool CX>
__global__ void __launch_bounds__(THREADS) dot_fast_kernel(DotArgs a) {
    prefetch_kernel_arguments<sizeof(DotArgs)>();
    constexpr int NV = CX ? 2 : (KV ? VEC : 1);   // accumulators per lane (complex: re, im)
    constexpr int LV = CX ? 2 : VEC;              // components per load of A
    constexpr int LB = CX ? 2 : (BB ? 1 : VEC);   // components per load of B
    constexpr int EC = CX ? 2 : 1;                // components per element
    extern __shared__ __align__(16) unsigned char smem_raw[];
    int64_t* rtab_a = reinterpret_cast<int64_t*>(smem_raw);                 // [rps] offsets of the serial indices in A
    int64_t* rtab_b = rtab_a + MAX_RTAB;                                    // ... and in B
    double* lds = reinterpret_cast<double*>(rtab_b + MAX_RTAB);             // [NV][THREADS]
    const int tid = threadIdx.x;
    const int r_begin = a.mode == 1 ? (int)blockIdx.y * a.rps : 0;
    const int r_count = a.mode == 2 ? 0 : (a.mode == 1 ? (a.r_total - r_begin < a.rps ? a.r_total - r_begin : a.rps) : a.r_total);
    int rot = a.rot_shift >= 0 && a.mode == 0 ? (int)((blockIdx.x >> a.rot_shift) % (uint32_t)r_count) : 0;
    // (a split range rotates each chunk by its number: vector x matrix 8192^2 f64 108.6 -> 101.3 us, f32 59.8 -> 51.4 us)
    if (a.mode == 1 && r_count > 0) rot = (int)(blockIdx.y % (uint32_t)r_count);
    for (int i = tid; i < r_count; i += THREADS) {
        int64_t lin = r_begin + (i + rot >= r_count ? i + rot - r_count : i + rot), oa = 0, ob = 0;
#pragma unroll
        for (int r = 0; r < MAXR; ++r)
            if (r < a.nr) {
                const int64_t q = lin / a.r_count[r], c = lin - q * a.r_count[r];
                oa += c * a.r_sa[r];
                ob += c * a.r_sb[r];
                lin = q;
            }
        rtab_a[i] = oa * EC;
        rtab_b[i] = ob * EC;
    }
    int64_t org_a = 0, org_b = 0, org_c = 0;
    {
        uint32_t bid = blockIdx.x;
        for (int g = 0; g < a.ng; ++g) {
            const uint32_t n = (uint32_t)a.g_count[g], q = bid / n;
            const int64_t c = (int64_t)(bid - q * n);
            bid = q;
            org_a += c * a.g_sa[g];
            org_b += c * a.g_sb[g];
            org_c += c * a.g_sc[g];
        }
    }
    int64_t toff_a = 0, toff_b = 0, toff_c = 0;
    bool writer = true;
#pragma unroll
    for (int t = 0; t < MAXT; ++t) {
        const int c = (tid >> a.t_shift[t]) & a.t_mask[t];
        toff_a += (int64_t)c * a.t_sa[t];
        toff_b += (int64_t)c * a.t_sb[t];
        if (a.t_red[t]) writer &= c == 0;
        else toff_c += (int64_t)c * a.t_sc[t];
    }
    __syncthreads();
    const R* A = reinterpret_cast<const R*>(a.a) + (org_a + toff_a) * EC;
    const R* B = reinterpret_cast<const R*>(a.b) + (org_b + toff_b) * EC;
    double acc[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) acc[j] = 0.0;

    constexpr int U = 4;   // two loads per step: eight in flight per thread
    RVec<R, LV> va[U];
    RVec<R, LB> vb[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (u < r_count) {
            va[u] = load_stream<R, LV>(A + rtab_a[u]);
            vb[u] = load_stream<R, LB>(B + rtab_b[u]);
        }
    for (int it = 0; it < r_count; it += U) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (it + u >= r_count) break;
            const RVec<R, LV> x = va[u];
            const RVec<R, LB> y = vb[u];
            if (it + U + u < r_count) {
                va[u] = load_stream<R, LV>(A + rtab_a[it + U + u]);
                vb[u] = load_stream<R, LB>(B + rtab_b[it + U + u]);
            }
            if constexpr (CX) {
                const double ar = (double)x.v[0], ai = (double)x.v[1], br = (double)y.v[0], bi = (double)y.v[1];
                acc[0] += ar * br - ai * bi;
                acc[1] += ar * bi + ai * br;
            } else if constexpr (KV) {
#pragma unroll
                for (int j = 0; j < VEC; ++j) acc[j] += (double)x.v[j] * (double)y.v[BB ? 0 : j];
            } else {
                double s = 0.0;
#pragma unroll
                for (int j = 0; j < VEC; ++j) s += (double)x.v[j] * (double)y.v[BB ? 0 : j];
                acc[0] += s;
            }
        }
    }
    if (a.mode == 2) {
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
            for (int j = 0; j < NV; ++j) acc[j] += src[j];
        }
    }
    // lanes that share an output: lane exchanges inside a wave, LDS across waves (thread-id bits 6 and 7)
#pragma unroll
    for (int b = 0; b < 6; ++b)
        if (a.red_bits & (1 << b)) {
#pragma unroll
            for (int j = 0; j < NV; ++j) acc[j] += __shfl_xor(acc[j], 1 << b);
        }
    if (a.red_bits & 0xc0) {
#pragma unroll
        for (int j = 0; j < NV; ++j) lds[j * THREADS + tid] = acc[j];
        __syncthreads();
        for (int b = 7; b >= 6; --b) {
            const int bit = 1 << b;
            if (a.red_bits & bit) {
                if (!(tid & bit)) {
#pragma unroll
                    for (int j = 0; j < NV; ++j) lds[j * THREADS + tid] += lds[j * THREADS + (tid | bit)];
                }
                __syncthreads();
            }
        }
#pragma unroll
        for (int j = 0; j < NV; ++j) acc[j] = lds[j * THREADS + tid];
    }
    if (!writer) return;
    if (a.mode == 1) {
        double* dst = a.partial + (((int64_t)blockIdx.y * a.nblocks + blockIdx.x) * THREADS + tid) * NV;
#pragma unroll
        for (int j = 0; j < NV; ++j) dst[j] = acc[j];
        return;
    }
    R* C = reinterpret_cast<R*>(a.c) + (org_c + toff_c) * EC;
    if constexpr (CX) {
        double rr = a.alpha_re * acc[0] - a.alpha_im * acc[1], ri = a.alpha_re * acc[1] + a.alpha_im * acc[0];
        if (a.use_beta) {
            const double cr = (double)C[0], ci = (double)C[1];
            rr += a.beta_re * cr - a.beta_im * ci;
            ri += a.beta_re * ci + a.beta_im * cr;
        }
        C[0] = (R)rr;
        C[1] = (R)ri;
    } else {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            R* dst = C + j * a.vc_stride;
            double r = a.alpha_re * acc[j];
            if (a.use_beta) r += a.beta_re * (double)*dst;
            *dst = (R)r;
        }
    }
}

int ceil_log2(int64_t n) {
    int l = 0;
    while (((int64_t)1 << l) < n) ++l;
    return l;
}

template <class R, int VEC, bool KV, bool BB, bool CX>
void launch_variant(const DotArgs& da, dim3 grid, hipStream_t st) {
    constexpr int NV = CX ? 2 : (KV ? VEC : 1);
    const size_t lds = (size_t)2 * MAX_RTAB * sizeof(int64_t) + (size_t)NV * THREADS * sizeof(double);
    TFH_LAUNCH_TIMED((dot_fast_kernel<R, VEC, KV, BB, CX>), grid, dim3(THREADS), lds, st, da);
}
template <class R>
void launch_real(const DotArgs& da, dim3 grid, int vec, bool kv, bool bb, hipStream_t st) {
    constexpr int V = 16 / sizeof(R);
    if (vec > 1) {
        if (kv) {
            if (bb) launch_variant<R, V, true, true, false>(da, grid, st);
            else launch_variant<R, V, true, false, false>(da, grid, st);
        } else {
            if (bb) launch_variant<R, V, false, true, false>(da, grid, st);
            else launch_variant<R, V, false, false, false>(da, grid, st);
        }
    } else {
        launch_variant<R, 1, true, false, false>(da, grid, st);
    }
}
void launch_any(int dtype, const DotArgs& da, dim3 grid, int vec, bool kv, bool bb, hipStream_t st) {
    switch (dtype) {
        case TFH_F32: launch_real<float>(da, grid, vec, kv, bb, st); break;
        case TFH_F64: launch_real<double>(da, grid, vec, kv, bb, st); break;
        case TFH_C64: launch_variant<float, 1, true, false, true>(da, grid, st); break;
        default: launch_variant<double, 1, true, false, true>(da, grid, st); break;
    }
}

}  // namespace

// kept / red: s[0] = A, s[1] = B, s[2] = C strides in elements (0 where an operand lacks the axis).  Returns true when
// the product was launched here (status then holds the outcome), false when the shape is not one this kernel tiles
// without partial tiles -- the caller then takes the tiled contraction kernels.
bool try_dot(int dtype, const void* a, const void* b, void* c, std::vector<Axis> kept, std::vector<Axis> red, Scalar alpha,
             Scalar beta, void* stream, int32_t& status) {
    status = TFH_OK;
    const bool cx = is_complex(dtype);
    const int ebytes = (int)dtype_size(dtype);
    if (!cx && (alpha.im != 0 || beta.im != 0)) return false;
    // A is the operand with more elements (its memory order decides the thread tile)
    auto elems = [&](int slot) {
        double n = 1;
        for (auto* grp : {&kept, &red})
            for (auto& x : *grp)
                if (x.s[slot] != 0) n *= (double)x.n;
        return n;
    };
    if (elems(1) > elems(0)) {
        std::swap(a, b);
        for (auto* grp : {&kept, &red})
            for (auto& x : *grp) std::swap(x.s[0], x.s[1]);
    }
    std::stable_sort(kept.begin(), kept.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[2]) > std::llabs(y.s[2]); });
    fuse_axes(kept, 3);
    auto key_a = [](const Axis& x) { return x.s[0] == 0 ? INT64_MAX : std::llabs(x.s[0]); };
    std::stable_sort(red.begin(), red.end(), [&](const Axis& x, const Axis& y) { return key_a(x) > key_a(y); });
    fuse_axes(red, 3);
    for (auto& x : kept)
        if (x.s[2] == 0) return false;
    struct Ax { Axis a; bool red; int tl; int64_t neff; };
    std::vector<Ax> all;
    for (auto& x : kept) all.push_back({x, false, 0, x.n});
    for (auto& x : red) all.push_back({x, true, 0, x.n});
    if (all.empty() || (int)all.size() > MAXG) return false;
    std::stable_sort(all.begin(), all.end(), [&](const Ax& x, const Ax& y) { return key_a(x.a) < key_a(y.a); });
    if (all[0].a.s[0] == 0) return false;   // A is a scalar: nothing to tile
    // 16-byte loads along A's contiguous axis (real types); B is contiguous there too, or has stride 0 there
    int vec = cx ? 1 : 16 / ebytes;
    bool bb = false;
    if (vec > 1) {
        const Ax& f = all[0];
        bool ok = f.a.s[0] == 1 && f.a.n % vec == 0 && ((uintptr_t)a % 16) == 0;
        for (size_t i = 1; i < all.size(); ++i) ok = ok && all[i].a.s[0] % vec == 0;
        if (f.a.s[1] == 0) {
            bb = true;
        } else {
            ok = ok && f.a.s[1] == 1 && ((uintptr_t)b % 16) == 0;
            for (size_t i = 1; i < all.size(); ++i) ok = ok && all[i].a.s[1] % vec == 0;
        }
        if (!all[0].red) ok = ok && true;
        if (!ok) { vec = 1; bb = false; }
    }
    const bool kv = !all[0].red;
    all[0].neff = all[0].a.n / vec;
    DotArgs da;
    std::memset(&da, 0, sizeof da);
    int bits = 8, shift = 0;
    for (size_t i = 0; i < all.size(); ++i) {
        Ax& x = all[i];
        if (bits == 0) break;
        int t = std::min(ceil_log2(x.neff), bits);
        while (t > 0 && x.neff % ((int64_t)1 << t) != 0) --t;   // no partial tiles
        if (t == 0) {
            if (x.neff == 1) continue;
            break;
        }
        if (da.nt == MAXT) break;
        x.tl = t;
        const int id = da.nt++;
        const int64_t mul = i == 0 ? vec : 1;
        da.t_shift[id] = shift;
        da.t_mask[id] = (1 << t) - 1;
        da.t_red[id] = x.red;
        da.t_sa[id] = x.a.s[0] * mul;
        da.t_sb[id] = x.a.s[1] * mul;
        da.t_sc[id] = x.a.s[2] * mul;
        if (x.red) da.red_bits |= da.t_mask[id] << shift;
        shift += t;
        bits -= t;
    }
    if (bits != 0) return false;
    int64_t blocks = 1, r_total = 1;
    for (size_t i = 0; i < all.size(); ++i) {
        const Ax& x = all[i];
        const int64_t text = (int64_t)1 << x.tl;
        const int64_t cnt = x.neff / text;
        if (cnt <= 1) continue;
        const int64_t mul = (i == 0 ? vec : 1) * text;
        if (x.red) {
            if (da.nr == MAXR) return false;
            da.r_count[da.nr] = cnt;
            da.r_sa[da.nr] = x.a.s[0] * mul;
            da.r_sb[da.nr] = x.a.s[1] * mul;
            ++da.nr;
            r_total *= cnt;
        } else {
            da.g_count[da.ng] = cnt;
            da.g_sa[da.ng] = x.a.s[0] * mul;
            da.g_sb[da.ng] = x.a.s[1] * mul;
            da.g_sc[da.ng] = x.a.s[2] * mul;
            ++da.ng;
            blocks *= cnt;
        }
    }
    if (blocks > 0x7fffffffll || r_total > 0x7fffffffll) return false;
    int64_t nchunks = 1, rps = r_total;
    if ((blocks < 512 && r_total >= 64) || r_total > MAX_RTAB) {   // (a serial range longer than the offset table is split as well)
        nchunks = std::max<int64_t>(1, std::min<int64_t>((2048 + blocks - 1) / blocks, r_total / 16));
        rps = (r_total + nchunks - 1) / nchunks;
        if (rps > MAX_RTAB) rps = MAX_RTAB;
        nchunks = (r_total + rps - 1) / rps;
        if (nchunks > 65535) return false;
    }
    const int nv = cx ? 2 : (kv ? vec : 1);
    da.r_total = (int32_t)r_total;
    // groups of 32 blocks start a serial axis that has a kept axis outside it at different indices (as in the reduction
    // kernel: blocks running in step would otherwise read addresses a large power of two apart at the same time);
    // a vector applied to a middle axis, [16,64,16,1024] x [64]: 28.6 -> 25.1 us
    da.rot_shift = -1;
    if (nchunks == 1 && r_total >= 4 && blocks >= 512 && da.nr >= 1 && da.ng >= 1) {
        int64_t serial_min = INT64_MAX, grid_max = 0;
        for (int r = 0; r < da.nr; ++r) serial_min = std::min<int64_t>(serial_min, std::llabs(da.r_sa[r]));
        for (int g = 0; g < da.ng; ++g) grid_max = std::max<int64_t>(grid_max, std::llabs(da.g_sa[g]));
        // (serial steps of at least 32 KB: the chunks of one contiguous row in a matrix-vector product gain nothing)
        if (grid_max > serial_min && serial_min * (int64_t)dtype_size(dtype) >= 32768) da.rot_shift = 5;
    }
    da.a = a;
    da.b = b;
    da.c = c;
    da.alpha_re = alpha.re; da.alpha_im = alpha.im; da.beta_re = beta.re; da.beta_im = beta.im;
    da.use_beta = !beta.is_zero();
    da.vc_stride = all[0].a.s[2];
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((uint32_t)blocks, (uint32_t)nchunks);
    if (nchunks > 1) {
        void* ws = nullptr;
        if (int32_t e = workspace(stream, (size_t)nchunks * (size_t)blocks * THREADS * nv * sizeof(double), &ws)) {
            status = e;
            return true;
        }
        da.mode = 1;
        da.nchunks = (int32_t)nchunks;
        da.rps = (int32_t)rps;
        da.nblocks = (int32_t)blocks;
        da.partial = (double*)ws;
    }
    const int prof = prof_begin(PROF_CONTRACT, stream);
    launch_any(dtype, da, grid, vec, kv, bb, st);
    prof_end(prof, stream);
    if (nchunks > 1) {
        da.mode = 2;
        launch_any(dtype, da, dim3((uint32_t)blocks), vec, kv, bb, st);
    }
    status = hip_check(hipGetLastError(), "dot kernel launch");
    return true;
}

}  // namespace tfh
