// k_gemm_tiny.hip -- a tiny operator applied to a long tensor: binary contractions (tenferro-prims/src/lib.rs:227-239)
// in which one operand has at most 8 free and at most 8 contracted indices and the other is long -- a gate on one or two
// legs of a state, a physical-index rotation of an MPS tensor: "ab,xby->xay".  A tile of MFMAs would compute a
// 64-row tile for two rows (0.3-0.5 TB/s on the tiled kernels); the work is a stream over the long operand: every thread
// takes one 16-byte vector of the long free index, loads it for each contracted index, and writes one vector per row
// of the operator, which sits in LDS.  HBM-bound: algorithmic bytes = sizeof(long operand) + sizeof(result).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <vector>

#include "internal.hpp"
#include "launch.hpp"

namespace tfh {
namespace {

constexpr int TINY_MAX = 8, TINY_NAX = 6, TINY_THREADS = 256;

struct TinyArgs {
    const void* S;   // the operator
    const void* T;   // the long operand
    void* C;
    int32_t ms, ks;  // free and contracted extent of the operator (fused), each <= TINY_MAX
    int32_t nax, use_beta;
    int32_t rows;                                          // C[n][m] with the rows m packed: results leave through an LDS tile
    int64_t total;                                         // vectors of the long free index
    int64_t next[TINY_NAX], nst[TINY_NAX], nsc[TINY_NAX];  // its axes, innermost first: extent (axis 0 in vectors), T and C strides
    int64_t s_off[TINY_MAX * TINY_MAX];                    // element offset of S[m][k]
    int64_t t_koff[TINY_MAX], c_moff[TINY_MAX];            // element offsets of contracted index k in T, of row m in C
    double alpha_re, alpha_im, beta_re, beta_im;
};

template <int BYTES> struct Raw;
template <> struct Raw<4> { typedef uint32_t type; };
template <> struct Raw<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct Raw<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

// R: component type; CX: complex elements; VEC: elements per access; KM: unroll bound of both small extents.
// ROWS (VEC = 1): the output is C[n][m] with the operator's rows m adjacent and packed (the acted-on leg comes last in
// the result).  A thread's ms results are then ms adjacent elements and neighbouring lanes are ms elements apart: stored
// directly, every store instruction touches 64 separate lines.  The block's 256 x ms results are one contiguous piece
// of C instead: they go through an LDS tile and leave as 16-byte stores in address order.
template <class R, bool CX, int VEC, int KM, bool ROWS = false>
__global__ void __launch_bounds__(TINY_THREADS) tiny_operator_kernel(TinyArgs a) {
    constexpr int NC = CX ? 2 : 1, W = VEC * NC;   // components per element, per access
    static_assert(!ROWS || VEC == 1, "");
    constexpr int ES = NC * (int)sizeof(R);         // bytes per element
    constexpr int TILE_PITCH = KM * ES + 16;        // bytes per thread's row of the tile (+16: lanes on different banks)
    __shared__ __align__(16) unsigned char tile[ROWS ? TINY_THREADS * TILE_PITCH : 16];
    typedef typename Raw<W * sizeof(R)>::type RawT;
    struct alignas(W * sizeof(R)) Vals { R v[W]; };
    __shared__ R s_op[TINY_MAX * TINY_MAX * NC];
    const int tid = threadIdx.x;
    if (tid < a.ms * a.ks) {
        const int m = tid / a.ks, k = tid - m * a.ks;
        const R* src = reinterpret_cast<const R*>(a.S) + a.s_off[m * TINY_MAX + k] * NC;
        s_op[(m * TINY_MAX + k) * NC] = src[0];
        if (CX) s_op[(m * TINY_MAX + k) * NC + 1] = src[1];
    }
    __syncthreads();
    int64_t v = (int64_t)blockIdx.x * TINY_THREADS + tid;
    if (v >= a.total) return;
    int64_t off_t = 0, off_c = 0;
#pragma unroll
    for (int d = 0; d < TINY_NAX; ++d)
        if (d < a.nax) {
            const int64_t q = v / a.next[d], c = (v - q * a.next[d]) * (d == 0 ? VEC : 1);
            v = q;
            off_t += c * a.nst[d];
            off_c += c * a.nsc[d];
        }
    const R* T = reinterpret_cast<const R*>(a.T) + off_t * NC;
    R* C = reinterpret_cast<R*>(a.C) + off_c * NC;
    Vals b[KM];
#pragma unroll
    for (int k = 0; k < KM; ++k)
        if (k < a.ks) b[k] = __builtin_bit_cast(Vals, __builtin_nontemporal_load(reinterpret_cast<const RawT*>(T + a.t_koff[k] * NC)));
    const R ar = (R)a.alpha_re, ai = (R)a.alpha_im, br = (R)a.beta_re, bi = (R)a.beta_im;
#pragma unroll
    for (int m = 0; m < KM; ++m) {
        if (m >= a.ms) break;
        Vals acc;
#pragma unroll
        for (int e = 0; e < W; ++e) acc.v[e] = R(0);
#pragma unroll
        for (int k = 0; k < KM; ++k)
            if (k < a.ks) {
                const R sr = s_op[(m * TINY_MAX + k) * NC], si = CX ? s_op[(m * TINY_MAX + k) * NC + 1] : R(0);
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if constexpr (CX) {
                        acc.v[2 * e] += sr * b[k].v[2 * e] - si * b[k].v[2 * e + 1];
                        acc.v[2 * e + 1] += sr * b[k].v[2 * e + 1] + si * b[k].v[2 * e];
                    } else {
                        acc.v[e] += sr * b[k].v[e];
                    }
                }
            }
        if constexpr (ROWS) {
            *reinterpret_cast<Vals*>(tile + tid * TILE_PITCH + m * ES) = acc;
            continue;
        }
        RawT* dst = reinterpret_cast<RawT*>(C + a.c_moff[m] * NC);
        Vals out, old;
        if (a.use_beta) old = __builtin_bit_cast(Vals, *dst);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            if constexpr (CX) {
                out.v[2 * e] = ar * acc.v[2 * e] - ai * acc.v[2 * e + 1];
                out.v[2 * e + 1] = ar * acc.v[2 * e + 1] + ai * acc.v[2 * e];
                if (a.use_beta) {
                    out.v[2 * e] += br * old.v[2 * e] - bi * old.v[2 * e + 1];
                    out.v[2 * e + 1] += br * old.v[2 * e + 1] + bi * old.v[2 * e];
                }
            } else {
                out.v[e] = ar * acc.v[e];
                if (a.use_beta) out.v[e] += br * old.v[e];
            }
        }
        __builtin_nontemporal_store(__builtin_bit_cast(RawT, out), dst);
    }
    if constexpr (ROWS) {
        __syncthreads();
        // the block's piece of C starts at thread 0's first element; 16-byte pieces of it in address order
        constexpr int PW = 16 / (int)sizeof(R);   // components per piece
        typedef typename Raw<16>::type Raw16;
        struct alignas(16) Piece { R v[PW]; };
        unsigned char* Cblk = reinterpret_cast<unsigned char*>(C) - (size_t)tid * a.ms * ES;
        const int row_bytes = a.ms * ES, pieces = TINY_THREADS * row_bytes / 16;
        for (int pc = tid; pc < pieces; pc += TINY_THREADS) {
            const int byte = pc * 16, row = byte / row_bytes, within = byte - row * row_bytes;
            const Piece x = *reinterpret_cast<const Piece*>(tile + row * TILE_PITCH + within);
            Raw16* dst = reinterpret_cast<Raw16*>(Cblk + byte);
            Piece out, old;
            if (a.use_beta) old = __builtin_bit_cast(Piece, *dst);
#pragma unroll
            for (int e = 0; e < PW; e += NC) {
                if constexpr (CX) {
                    out.v[e] = ar * x.v[e] - ai * x.v[e + 1];
                    out.v[e + 1] = ar * x.v[e + 1] + ai * x.v[e];
                    if (a.use_beta) {
                        out.v[e] += br * old.v[e] - bi * old.v[e + 1];
                        out.v[e + 1] += br * old.v[e + 1] + bi * old.v[e];
                    }
                } else {
                    out.v[e] = ar * x.v[e];
                    if (a.use_beta) out.v[e] += br * old.v[e];
                }
            }
            __builtin_nontemporal_store(__builtin_bit_cast(Raw16, out), dst);
        }
    }
}

template <class R, bool CX, int VEC>
void launch_km(const TinyArgs& ta, int km, dim3 grid, hipStream_t st) {
    if (km <= 2) TFH_LAUNCH_TIMED((tiny_operator_kernel<R, CX, VEC, 2>), grid, dim3(TINY_THREADS), 0, st, ta);
    else if (km <= 4) TFH_LAUNCH_TIMED((tiny_operator_kernel<R, CX, VEC, 4>), grid, dim3(TINY_THREADS), 0, st, ta);
    else TFH_LAUNCH_TIMED((tiny_operator_kernel<R, CX, VEC, 8>), grid, dim3(TINY_THREADS), 0, st, ta);
}
template <class R, bool CX>
void launch_vec(const TinyArgs& ta, bool vec, int km, dim3 grid, hipStream_t st) {
    constexpr int VMAX = 16 / (int)(sizeof(R) * (CX ? 2 : 1));
    if (ta.rows) {
        if (km <= 4) TFH_LAUNCH_TIMED((tiny_operator_kernel<R, CX, 1, 4, true>), grid, dim3(TINY_THREADS), 0, st, ta);
        else TFH_LAUNCH_TIMED((tiny_operator_kernel<R, CX, 1, 8, true>), grid, dim3(TINY_THREADS), 0, st, ta);
    } else if (vec && VMAX > 1) launch_km<R, CX, VMAX>(ta, km, grid, st);
    else launch_km<R, CX, 1>(ta, km, grid, st);
}

int64_t prod_of(const std::vector<Axis>& g) {
    int64_t p = 1;
    for (auto& x : g) p *= x.n;
    return p;
}

}  // namespace

bool try_tiny_operator(int dtype, const void* a, const void* b, void* c, const ContractAxes& ax, Scalar alpha, Scalar beta,
                       void* stream, int32_t& status) {
    status = TFH_OK;
    if (!ax.batch.empty() && prod_of(ax.batch) != 1) return false;
    const int64_t M = prod_of(ax.M), N = prod_of(ax.N), K = prod_of(ax.K);
    if (K > TINY_MAX || K < 1) return false;
    // which operand is the operator: slot = its stride slot in the axes (0 = A, 1 = B)
    int sslot;
    if (M <= TINY_MAX && N >= 65536) sslot = 0;
    else if (N <= TINY_MAX && M >= 65536) sslot = 1;
    else return false;
    const int tslot = 1 - sslot;
    const std::vector<Axis>& small = sslot == 0 ? ax.M : ax.N;
    const std::vector<Axis>& big = sslot == 0 ? ax.N : ax.M;
    const void* S = sslot == 0 ? a : b;
    const void* T = sslot == 0 ? b : a;
    TinyArgs ta;
    std::memset(&ta, 0, sizeof ta);
    ta.S = S; ta.T = T; ta.C = c;
    ta.ms = (int32_t)prod_of(small);
    ta.ks = (int32_t)K;
    // fused small indices, last axis fastest
    auto enumerate = [](const std::vector<Axis>& grp, int slot, int64_t* out) {
        const int64_t total = prod_of(grp);
        for (int64_t i = 0; i < total; ++i) {
            int64_t lin = i, off = 0;
            for (size_t d = grp.size(); d-- > 0;) {
                off += (lin % grp[d].n) * grp[d].s[slot];
                lin /= grp[d].n;
            }
            out[i] = off;
        }
    };
    int64_t s_m[TINY_MAX] = {0}, s_k[TINY_MAX] = {0};
    enumerate(small, sslot, s_m);
    enumerate(small, 2, ta.c_moff);
    enumerate(ax.K, sslot, s_k);
    enumerate(ax.K, tslot, ta.t_koff);
    for (int m = 0; m < ta.ms; ++m)
        for (int k = 0; k < ta.ks; ++k) ta.s_off[m * TINY_MAX + k] = s_m[m] + s_k[k];
    // the long free index: axes by C stride, merged where contiguous in T and in C
    std::vector<Axis> nx;
    for (auto& x : big) nx.push_back(Axis{x.n, {x.s[tslot], x.s[2], 0}, x.label});
    std::stable_sort(nx.begin(), nx.end(), [](const Axis& x, const Axis& y) { return std::llabs(x.s[1]) > std::llabs(y.s[1]); });
    fuse_axes(nx, 2);
    if (nx.empty() || (int)nx.size() > TINY_NAX) return false;
    std::reverse(nx.begin(), nx.end());   // innermost first
    const bool cx = is_complex(dtype);
    const int ebytes = (int)dtype_size(dtype), vmax = 16 / ebytes;
    bool vec = vmax > 1 && nx[0].s[0] == 1 && nx[0].s[1] == 1 && nx[0].n % vmax == 0 && (uintptr_t)T % 16 == 0 && (uintptr_t)c % 16 == 0;
    for (size_t d = 1; d < nx.size(); ++d) vec = vec && nx[d].s[0] % vmax == 0 && nx[d].s[1] % vmax == 0;
    for (int k = 0; k < ta.ks; ++k) vec = vec && ta.t_koff[k] % vmax == 0;
    for (int m = 0; m < ta.ms; ++m) vec = vec && ta.c_moff[m] % vmax == 0;
    // C[n][m] with packed rows of m: whole blocks of 256 n inside the innermost long axis, rows of whole 16-byte pieces
    bool rows = !vec && ta.ms >= 3 && nx[0].s[1] == ta.ms && nx[0].n % TINY_THREADS == 0 && (uintptr_t)c % 16 == 0 &&
                (int64_t)ta.ms * ebytes % 16 == 0;
    for (int m = 0; m < ta.ms; ++m) rows = rows && ta.c_moff[m] == m;
    for (size_t d = 1; d < nx.size(); ++d) rows = rows && nx[d].s[1] * ebytes % 16 == 0;
    ta.rows = rows;
    const int v = vec ? vmax : 1;
    ta.nax = (int32_t)nx.size();
    ta.total = 1;
    for (size_t d = 0; d < nx.size(); ++d) {
        ta.next[d] = d == 0 ? nx[d].n / v : nx[d].n;
        ta.nst[d] = nx[d].s[0];
        ta.nsc[d] = nx[d].s[1];
        ta.total *= ta.next[d];
    }
    const int64_t blocks = (ta.total + TINY_THREADS - 1) / TINY_THREADS;
    if (blocks > 0x7fffffffll) return false;
    ta.alpha_re = alpha.re; ta.alpha_im = alpha.im; ta.beta_re = beta.re; ta.beta_im = beta.im;
    ta.use_beta = !beta.is_zero();
    const int km = std::max(ta.ms, ta.ks);
    const dim3 grid((uint32_t)blocks);
    hipStream_t st = (hipStream_t)stream;
    const int prof = prof_begin(PROF_CONTRACT, stream);
    switch (dtype) {
        case TFH_F32: launch_vec<float, false>(ta, vec, km, grid, st); break;
        case TFH_F64: launch_vec<double, false>(ta, vec, km, grid, st); break;
        case TFH_C64: launch_vec<float, true>(ta, vec, km, grid, st); break;
        default: launch_vec<double, true>(ta, vec, km, grid, st); break;
    }
    (void)cx;
    prof_end(prof, stream);
    status = hip_check(hipGetLastError(), "contraction kernel launch");
    return true;
}

}  // namespace tfh
