// tfo_oracle.cpp -- CPU restatement of tenferro's tensor primitives (see tfo_oracle.h).
// TEST INFRASTRUCTURE ONLY: the checker for the HIP backend and the timed CPU baseline.
// Parity with a reference implementation is unpinned -- the reference has none
// (tenferro-prims/src/lib.rs:419-439 are todo!()); each function follows the documented
// formula it cites and is pinned by numpy cross-checks, closed forms and brute force in tests/.
#include "tfo_oracle.h"

#include <omp.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace {

thread_local std::string g_msg;
int g_threads = 0;

int fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_msg = buf;
    return code;
}
constexpr int E_SHAPE = -1, E_RANK = -2, E_ARG = -6;

int nthreads() { return g_threads > 0 ? g_threads : omp_get_max_threads(); }

inline bool is_complex(int dt) { return dt == TFO_C64 || dt == TFO_C128; }

// One logical loop axis with a stride per participating tensor (0 = tensor does not carry it).
struct Axis {
    uint32_t label;
    int64_t n;
    int64_t s[3];
};

int find_label(const uint32_t* modes, int n, uint32_t l) {
    for (int i = 0; i < n; ++i)
        if (modes[i] == l) return i;
    return -1;
}
bool has_repeats(const uint32_t* modes, int n) {
    for (int i = 0; i < n; ++i)
        for (int j = i + 1; j < n; ++j)
            if (modes[i] == modes[j]) return true;
    return false;
}
int64_t product(const std::vector<Axis>& ax) {
    int64_t p = 1;
    for (auto& a : ax) p *= a.n;
    return p;
}
// Offset of linear index `lin` (last axis fastest) for tensor slot t.
inline int64_t offset_of(const std::vector<Axis>& ax, int64_t lin, int t) {
    int64_t off = 0;
    for (int d = (int)ax.size() - 1; d >= 0; --d) {
        int64_t q = lin / ax[d].n;
        off += (lin - q * ax[d].n) * ax[d].s[t];
        lin = q;
    }
    return off;
}
// Table of offsets for a whole axis group (last axis fastest).
std::vector<int64_t> offset_table(const std::vector<Axis>& ax, int t) {
    int64_t n = product(ax);
    std::vector<int64_t> tab((size_t)n);
    std::vector<int64_t> idx(ax.size(), 0);
    int64_t off = 0;
    for (int64_t i = 0; i < n; ++i) {
        tab[(size_t)i] = off;
        for (int d = (int)ax.size() - 1; d >= 0; --d) {
            off += ax[d].s[t];
            if (++idx[d] < ax[d].n) break;
            off -= ax[d].s[t] * ax[d].n;
            idx[d] = 0;
        }
    }
    return tab;
}

// ---- scalar helpers: R = float/double, CX = interleaved complex --------------------------------
template <class R, bool CX>
struct Sc {
    R re, im;
    static Sc load(const void* p) {
        const R* r = (const R*)p;
        return {r[0], CX ? r[1] : R(0)};
    }
    bool is_zero() const { return re == R(0) && im == R(0); }
    bool is_one() const { return re == R(1) && im == R(0); }
};
template <class R, bool CX>
inline void axpby(R* dst, const Sc<R, CX>& al, R xr, R xi, const Sc<R, CX>& be) {
    // dst = al*x + be*dst ; be == 0 overwrites without reading dst (BLAS rule,
    // tenferro-prims/src/lib.rs:306-309 "(overwrite)")
    if (CX) {
        R rr = al.re * xr - al.im * xi, ri = al.re * xi + al.im * xr;
        if (!be.is_zero()) {
            R dr = dst[0], di = dst[1];
            rr += be.re * dr - be.im * di;
            ri += be.re * di + be.im * dr;
        }
        dst[0] = rr;
        dst[1] = ri;
    } else {
        R r = al.re * xr;
        if (!be.is_zero()) r += be.re * dst[0];
        dst[0] = r;
    }
}

// ================================================================================================
// Permute
// ================================================================================================
template <class R, bool CX>
int permute_impl(const void* alpha, const tfo_view* a, const uint32_t* ma, const void* beta, tfo_view* b,
                 const uint32_t* mb) {
    constexpr int NC = CX ? 2 : 1;
    auto al = Sc<R, CX>::load(alpha);
    auto be = Sc<R, CX>::load(beta);
    std::vector<Axis> ax;
    for (int d = 0; d < b->rank; ++d) {
        int j = find_label(ma, a->rank, mb[d]);
        if (j < 0) return fail(E_ARG, "permute: output mode %u not among input modes", mb[d]);
        if (a->dims[j] != b->dims[d]) return fail(E_SHAPE, "permute: extent of mode %u differs", mb[d]);
        ax.push_back({mb[d], b->dims[d], {a->strides[j], b->strides[d], 0}});
    }
    const R* A = (const R*)a->base + a->offset * NC;
    R* B = (R*)b->base + b->offset * NC;
    const bool copy = al.is_one() && be.is_zero();
    int64_t total = product(ax);
    if (total == 0) return 0;
    if (ax.empty()) {
        if (copy) memcpy(B, A, sizeof(R) * NC);
        else axpby<R, CX>(B, al, A[0], CX ? A[1] : R(0), be);
        return 0;
    }
    // innermost two loops: the axis fastest in the output and the axis fastest in the input
    int ao = 0, ai = 0;
    for (int d = 0; d < (int)ax.size(); ++d) {
        if (std::llabs(ax[d].s[1]) < std::llabs(ax[ao].s[1]) || ax[ao].n == 1) ao = d;
        if (std::llabs(ax[d].s[0]) < std::llabs(ax[ai].s[0]) || ax[ai].n == 1) ai = d;
    }
    std::vector<Axis> outer;
    for (int d = 0; d < (int)ax.size(); ++d)
        if (d != ao && d != ai) outer.push_back(ax[d]);
    Axis X = ax[ao], Y = ax[ai];
    bool two = ao != ai;
    int64_t nouter = product(outer);
    constexpr int64_t T = 16;
#pragma omp parallel for schedule(static) num_threads(nthreads())
    for (int64_t o = 0; o < nouter; ++o) {
        int64_t oa = offset_of(outer, o, 0), ob = offset_of(outer, o, 1);
        if (!two) {
            for (int64_t x = 0; x < X.n; ++x) {
                const R* src = A + (oa + x * X.s[0]) * NC;
                R* dst = B + (ob + x * X.s[1]) * NC;
                if (copy) {
                    dst[0] = src[0];
                    if (CX) dst[1] = src[1];
                } else
                    axpby<R, CX>(dst, al, src[0], CX ? src[1] : R(0), be);
            }
        } else {
            for (int64_t y0 = 0; y0 < Y.n; y0 += T)
                for (int64_t x0 = 0; x0 < X.n; x0 += T)
                    for (int64_t y = y0; y < std::min(Y.n, y0 + T); ++y)
                        for (int64_t x = x0; x < std::min(X.n, x0 + T); ++x) {
                            const R* src = A + (oa + x * X.s[0] + y * Y.s[0]) * NC;
                            R* dst = B + (ob + x * X.s[1] + y * Y.s[1]) * NC;
                            if (copy) {
                                dst[0] = src[0];
                                if (CX) dst[1] = src[1];
                            } else
                                axpby<R, CX>(dst, al, src[0], CX ? src[1] : R(0), be);
                        }
        }
    }
    return 0;
}

// ================================================================================================
// Reduce
// ================================================================================================
template <class R, bool CX>
int reduce_impl(const void* alpha, const tfo_view* a, const uint32_t* ma, const void* beta, tfo_view* c,
                const uint32_t* mc, int op) {
    constexpr int NC = CX ? 2 : 1;
    if (CX && op != TFO_SUM) return fail(E_ARG, "reduce: max/min are undefined for complex types");
    if (has_repeats(ma, a->rank) || has_repeats(mc, c->rank)) return fail(E_ARG, "reduce: repeated mode label");
    auto al = Sc<R, CX>::load(alpha);
    auto be = Sc<R, CX>::load(beta);
    std::vector<Axis> kept, red;
    for (int d = 0; d < c->rank; ++d) {
        int j = find_label(ma, a->rank, mc[d]);
        if (j < 0) return fail(E_ARG, "reduce: output mode %u is not an input mode", mc[d]);
        if (a->dims[j] != c->dims[d]) return fail(E_SHAPE, "reduce: extent of mode %u differs", mc[d]);
        kept.push_back({mc[d], c->dims[d], {a->strides[j], c->strides[d], 0}});
    }
    for (int j = 0; j < a->rank; ++j)
        if (find_label(mc, c->rank, ma[j]) < 0) red.push_back({ma[j], a->dims[j], {a->strides[j], 0, 0}});
    const R* A = (const R*)a->base + a->offset * NC;
    R* C = (R*)c->base + c->offset * NC;
    int64_t nk = product(kept), nr = product(red);
    if (nk == 0) return 0;
    // vector axis: the kept axis with the smallest input stride (contiguous rows when possible)
    int vi = -1;
    for (int d = 0; d < (int)kept.size(); ++d)
        if (vi < 0 || std::llabs(kept[d].s[0]) < std::llabs(kept[vi].s[0])) vi = d;
    Axis V = vi >= 0 ? kept[vi] : Axis{0, 1, {0, 0, 0}};
    std::vector<Axis> outer;
    for (int d = 0; d < (int)kept.size(); ++d)
        if (d != vi) outer.push_back(kept[d]);
    int64_t nouter = product(outer);
    std::vector<int64_t> rtab = offset_table(red, 0);
    const double init = op == TFO_SUM ? 0.0 : (op == TFO_MAX ? -INFINITY : INFINITY);
#pragma omp parallel num_threads(nthreads())
    {
        std::vector<double> acc((size_t)V.n * NC);
#pragma omp for schedule(static)
        for (int64_t o = 0; o < nouter; ++o) {
            int64_t oa = offset_of(outer, o, 0), oc = offset_of(outer, o, 1);
            std::fill(acc.begin(), acc.end(), init);
            for (int64_t r = 0; r < nr; ++r) {
                const R* row = A + (oa + rtab[(size_t)r]) * NC;
                if (op == TFO_SUM) {
                    for (int64_t v = 0; v < V.n; ++v) {
                        acc[(size_t)v * NC] += (double)row[v * V.s[0] * NC];
                        if (CX) acc[(size_t)v * NC + 1] += (double)row[v * V.s[0] * NC + 1];
                    }
                } else if (op == TFO_MAX) {
                    for (int64_t v = 0; v < V.n; ++v) acc[(size_t)v] = std::max(acc[(size_t)v], (double)row[v * V.s[0]]);
                } else {
                    for (int64_t v = 0; v < V.n; ++v) acc[(size_t)v] = std::min(acc[(size_t)v], (double)row[v * V.s[0]]);
                }
            }
            for (int64_t v = 0; v < V.n; ++v) {
                R* dst = C + (oc + v * V.s[1]) * NC;
                axpby<R, CX>(dst, al, (R)acc[(size_t)v * NC], CX ? (R)acc[(size_t)v * NC + 1] : R(0), be);
            }
        }
    }
    (void)nk;
    return 0;
}

// ================================================================================================
// Contract: mode classification shared by the blocked and the brute-force evaluator
// ================================================================================================
struct ContractModes {
    std::vector<Axis> batch, M, N, K;  // s[0]=A, s[1]=B, s[2]=C
};

int classify(const tfo_view* a, const uint32_t* ma, const tfo_view* b, const uint32_t* mb, const tfo_view* c,
             const uint32_t* mc, ContractModes& out) {
    if (has_repeats(ma, a->rank) || has_repeats(mb, b->rank) || has_repeats(mc, c->rank))
        return fail(E_ARG, "contract: repeated mode label inside one operand");
    std::set<uint32_t> seen;
    auto add = [&](uint32_t l) -> int {
        if (!seen.insert(l).second) return 0;
        int ia = find_label(ma, a->rank, l), ib = find_label(mb, b->rank, l), ic = find_label(mc, c->rank, l);
        int64_t n = ia >= 0 ? a->dims[ia] : (ib >= 0 ? b->dims[ib] : c->dims[ic]);
        if ((ia >= 0 && a->dims[ia] != n) || (ib >= 0 && b->dims[ib] != n) || (ic >= 0 && c->dims[ic] != n))
            return fail(E_SHAPE, "contract: extent of mode %u differs between operands", l);
        if (ia < 0 && ib < 0) return fail(E_ARG, "contract: output mode %u appears in no input", l);
        Axis ax{l, n, {ia >= 0 ? a->strides[ia] : 0, ib >= 0 ? b->strides[ib] : 0, ic >= 0 ? c->strides[ic] : 0}};
        // modes in inputs and output are batch/free, modes only in inputs are contracted
        // (tenferro-prims/src/lib.rs:136-138)
        if (ic >= 0) {
            if (ia >= 0 && ib >= 0) out.batch.push_back(ax);
            else if (ia >= 0) out.M.push_back(ax);
            else out.N.push_back(ax);
        } else
            out.K.push_back(ax);  // summed; an input that lacks it has stride 0 (sum of a broadcast)
        return 0;
    };
    for (int d = 0; d < c->rank; ++d)
        if (int e = add(mc[d])) return e;
    for (int d = 0; d < a->rank; ++d)
        if (int e = add(ma[d])) return e;
    for (int d = 0; d < b->rank; ++d)
        if (int e = add(mb[d])) return e;
    return 0;
}

// Micro-kernel: acc[MR][NR] over kc steps.  Ap: [kc][MR] (k-major), Bp: [kc][NR].
constexpr int MR = 6, NR = 16;
template <class R>
__attribute__((target_clones("avx512f", "avx2", "default"))) void micro_real(int64_t kc, const R* __restrict Ap,
                                                                              const R* __restrict Bp,
                                                                              double* __restrict Cacc, int64_t ldc) {
    R acc[MR][NR] = {};
    for (int64_t k = 0; k < kc; ++k) {
        const R* bp = Bp + k * NR;
        const R* ap = Ap + k * MR;
        for (int i = 0; i < MR; ++i) {
            R av = ap[i];
#pragma omp simd
            for (int j = 0; j < NR; ++j) acc[i][j] += av * bp[j];
        }
    }
    for (int i = 0; i < MR; ++i)
        for (int j = 0; j < NR; ++j) Cacc[i * ldc + j] += (double)acc[i][j];
}
// complex: planes (re, im) packed as Ap: [kc][2][MR], Bp: [kc][2][NR]; Cacc interleaved planes [MR][2][ldc]
constexpr int MRC = 3;
template <class R>
__attribute__((target_clones("avx512f", "avx2", "default"))) void micro_cplx(int64_t kc, const R* __restrict Ap,
                                                                              const R* __restrict Bp,
                                                                              double* __restrict Cr,
                                                                              double* __restrict Ci, int64_t ldc) {
    R ar_[MRC][NR] = {}, ai_[MRC][NR] = {};
    for (int64_t k = 0; k < kc; ++k) {
        const R* br = Bp + k * 2 * NR;
        const R* bi = br + NR;
        const R* ap = Ap + k * 2 * MRC;
        for (int i = 0; i < MRC; ++i) {
            R xr = ap[i], xi = ap[MRC + i];
#pragma omp simd
            for (int j = 0; j < NR; ++j) {
                ar_[i][j] += xr * br[j] - xi * bi[j];
                ai_[i][j] += xr * bi[j] + xi * br[j];
            }
        }
    }
    for (int i = 0; i < MRC; ++i)
        for (int j = 0; j < NR; ++j) {
            Cr[i * ldc + j] += (double)ar_[i][j];
            Ci[i * ldc + j] += (double)ai_[i][j];
        }
}

template <class R, bool CX>
int contract_impl(const void* alpha, const tfo_view* a, const uint32_t* ma, const tfo_view* b, const uint32_t* mb,
                  const void* beta, tfo_view* c, const uint32_t* mc) {
    constexpr int NC = CX ? 2 : 1;
    constexpr int mr = CX ? MRC : MR;
    ContractModes cm;
    if (int e = classify(a, ma, b, mb, c, mc, cm)) return e;
    auto al = Sc<R, CX>::load(alpha);
    auto be = Sc<R, CX>::load(beta);
    const R* A = (const R*)a->base + a->offset * NC;
    const R* B = (const R*)b->base + b->offset * NC;
    R* C = (R*)c->base + c->offset * NC;
    const int64_t nb = product(cm.batch), M = product(cm.M), N = product(cm.N), K = product(cm.K);
    if (nb * M * N == 0) return 0;
    auto aM = offset_table(cm.M, 0), cM = offset_table(cm.M, 2);
    auto bN = offset_table(cm.N, 1), cN = offset_table(cm.N, 2);
    auto aK = offset_table(cm.K, 0), bK = offset_table(cm.K, 1);
    auto aB = offset_table(cm.batch, 0), bB = offset_table(cm.batch, 1), cB = offset_table(cm.batch, 2);
    const int64_t Npan = (N + NR - 1) / NR, Np = Npan * NR;
    const int64_t KC = 256;
    const int64_t MC = mr * (CX ? 16 : 8);  // rows per work item
    const int64_t nmb = (M + MC - 1) / MC;
    // B packed once per batch entry: panels [Npan][K][NC][NR], zero padded
    std::vector<R> Bp((size_t)Npan * (size_t)std::max<int64_t>(K, 1) * NC * NR);
    for (int64_t bi = 0; bi < nb; ++bi) {
#pragma omp parallel for schedule(static) num_threads(nthreads())
        for (int64_t p = 0; p < Npan; ++p)
            for (int64_t k = 0; k < K; ++k) {
                R* dst = Bp.data() + ((size_t)p * K + k) * NC * NR;
                for (int j = 0; j < NR; ++j) {
                    int64_t n = p * NR + j;
                    if (n < N) {
                        const R* src = B + (bB[(size_t)bi] + bK[(size_t)k] + bN[(size_t)n]) * NC;
                        dst[j] = src[0];
                        if (CX) dst[NR + j] = src[1];
                    } else {
                        dst[j] = 0;
                        if (CX) dst[NR + j] = 0;
                    }
                }
            }
#pragma omp parallel num_threads(nthreads())
        {
            std::vector<R> Ap((size_t)MC * KC * NC);
            std::vector<double> Cacc((size_t)MC * Np * NC);
#pragma omp for schedule(dynamic, 1)
            for (int64_t mb_ = 0; mb_ < nmb; ++mb_) {
                int64_t m0 = mb_ * MC, mcnt = std::min(MC, M - m0);
                int64_t mpan = (mcnt + mr - 1) / mr;
                std::fill(Cacc.begin(), Cacc.end(), 0.0);
                for (int64_t k0 = 0; k0 < K; k0 += KC) {
                    int64_t kc = std::min(KC, K - k0);
                    // pack A rows m0.. into micro-panels [mpan][kc][NC][mr]
                    for (int64_t ip = 0; ip < mpan; ++ip)
                        for (int64_t k = 0; k < kc; ++k) {
                            R* dst = Ap.data() + ((size_t)ip * kc + k) * NC * mr;
                            for (int i = 0; i < mr; ++i) {
                                int64_t m = m0 + ip * mr + i;
                                if (m < M) {
                                    const R* src = A + (aB[(size_t)bi] + aM[(size_t)m] + aK[(size_t)(k0 + k)]) * NC;
                                    dst[i] = src[0];
                                    if (CX) dst[mr + i] = src[1];
                                } else {
                                    dst[i] = 0;
                                    if (CX) dst[mr + i] = 0;
                                }
                            }
                        }
                    for (int64_t p = 0; p < Npan; ++p) {
                        const R* bp = Bp.data() + ((size_t)p * K + k0) * NC * NR;
                        for (int64_t ip = 0; ip < mpan; ++ip) {
                            const R* ap = Ap.data() + (size_t)ip * kc * NC * mr;
                            if (CX) {
                                double* cr = Cacc.data() + ((size_t)ip * mr) * 2 * Np + p * NR;
                                micro_cplx<R>(kc, ap, bp, cr, cr + Np, 2 * Np);
                            } else {
                                micro_real<R>(kc, ap, bp, Cacc.data() + ((size_t)ip * mr) * Np + p * NR, Np);
                            }
                        }
                    }
                }
                for (int64_t i = 0; i < mcnt; ++i)
                    for (int64_t n = 0; n < N; ++n) {
                        R* dst = C + (cB[(size_t)bi] + cM[(size_t)(m0 + i)] + cN[(size_t)n]) * NC;
                        if (CX)
                            axpby<R, CX>(dst, al, (R)Cacc[(size_t)i * 2 * Np + n], (R)Cacc[(size_t)i * 2 * Np + Np + n], be);
                        else
                            axpby<R, CX>(dst, al, (R)Cacc[(size_t)i * Np + n], R(0), be);
                    }
            }
        }
    }
    return 0;
}

template <class R, bool CX>
int contract_naive_impl(const void* alpha, const tfo_view* a, const uint32_t* ma, const tfo_view* b,
                        const uint32_t* mb, const void* beta, tfo_view* c, const uint32_t* mc) {
    constexpr int NC = CX ? 2 : 1;
    ContractModes cm;
    if (int e = classify(a, ma, b, mb, c, mc, cm)) return e;
    auto al = Sc<R, CX>::load(alpha);
    auto be = Sc<R, CX>::load(beta);
    const R* A = (const R*)a->base + a->offset * NC;
    const R* B = (const R*)b->base + b->offset * NC;
    R* C = (R*)c->base + c->offset * NC;
    std::vector<Axis> outer = cm.batch;
    outer.insert(outer.end(), cm.M.begin(), cm.M.end());
    outer.insert(outer.end(), cm.N.begin(), cm.N.end());
    int64_t no = product(outer), nk = product(cm.K);
    for (int64_t o = 0; o < no; ++o) {
        int64_t oa = offset_of(outer, o, 0), ob = offset_of(outer, o, 1), oc = offset_of(outer, o, 2);
        long double sr = 0, si = 0;
        for (int64_t k = 0; k < nk; ++k) {
            const R* x = A + (oa + offset_of(cm.K, k, 0)) * NC;
            const R* y = B + (ob + offset_of(cm.K, k, 1)) * NC;
            if (CX) {
                sr += (long double)x[0] * y[0] - (long double)x[1] * y[1];
                si += (long double)x[0] * y[1] + (long double)x[1] * y[0];
            } else
                sr += (long double)x[0] * y[0];
        }
        axpby<R, CX>(C + oc * NC, al, (R)sr, (R)si, be);
    }
    return 0;
}

// ================================================================================================
// ElementwiseMul, conj
// ================================================================================================
template <class R, bool CX>
int emul_impl(const void* alpha, const tfo_view* a, const tfo_view* b, const void* beta, tfo_view* c) {
    constexpr int NC = CX ? 2 : 1;
    if (a->rank != c->rank || b->rank != c->rank) return fail(E_RANK, "elementwise_mul: ranks differ");
    std::vector<Axis> ax;
    for (int d = 0; d < c->rank; ++d) {
        if (a->dims[d] != c->dims[d] || b->dims[d] != c->dims[d]) return fail(E_SHAPE, "elementwise_mul: dims differ");
        ax.push_back({(uint32_t)d, c->dims[d], {a->strides[d], b->strides[d], c->strides[d]}});
    }
    auto al = Sc<R, CX>::load(alpha);
    auto be = Sc<R, CX>::load(beta);
    const R* A = (const R*)a->base + a->offset * NC;
    const R* B = (const R*)b->base + b->offset * NC;
    R* C = (R*)c->base + c->offset * NC;
    int64_t n = product(ax);
#pragma omp parallel for schedule(static) num_threads(nthreads())
    for (int64_t i = 0; i < n; ++i) {
        const R* x = A + offset_of(ax, i, 0) * NC;
        const R* y = B + offset_of(ax, i, 1) * NC;
        R pr, pi = 0;
        if (CX) {
            pr = x[0] * y[0] - x[1] * y[1];
            pi = x[0] * y[1] + x[1] * y[0];
        } else
            pr = x[0] * y[0];
        axpby<R, CX>(C + offset_of(ax, i, 2) * NC, al, pr, pi, be);
    }
    return 0;
}

template <class R, bool CX>
int conj_impl(const tfo_view* in, tfo_view* out) {
    constexpr int NC = CX ? 2 : 1;
    if (in->rank != out->rank) return fail(E_RANK, "conj: ranks differ");
    std::vector<Axis> ax;
    for (int d = 0; d < in->rank; ++d) {
        if (in->dims[d] != out->dims[d]) return fail(E_SHAPE, "conj: dims differ");
        ax.push_back({(uint32_t)d, in->dims[d], {in->strides[d], out->strides[d], 0}});
    }
    const R* A = (const R*)in->base + in->offset * NC;
    R* B = (R*)out->base + out->offset * NC;
    int64_t n = product(ax);
#pragma omp parallel for schedule(static) num_threads(nthreads())
    for (int64_t i = 0; i < n; ++i) {
        const R* x = A + offset_of(ax, i, 0) * NC;
        R* y = B + offset_of(ax, i, 1) * NC;
        y[0] = x[0];
        if (CX) y[1] = -x[1];
    }
    return 0;
}

// ================================================================================================
// einsum by brute force
// ================================================================================================
template <class R, bool CX>
int einsum_naive_impl(int n_in, const tfo_view* in, const uint32_t* labels, const int32_t* ranks,
                      const uint32_t* ol, int n_out, const void* alpha, const void* beta, tfo_view* out) {
    constexpr int NC = CX ? 2 : 1;
    auto al = Sc<R, CX>::load(alpha);
    auto be = Sc<R, CX>::load(beta);
    std::map<uint32_t, int64_t> ext;
    {
        const uint32_t* p = labels;
        for (int t = 0; t < n_in; ++t) {
            if (in[t].rank != ranks[t]) return fail(E_RANK, "einsum: operand %d has rank %d, subscripts say %d", t, in[t].rank, ranks[t]);
            for (int d = 0; d < ranks[t]; ++d) {
                auto it = ext.find(p[d]);
                if (it == ext.end()) ext[p[d]] = in[t].dims[d];
                else if (it->second != in[t].dims[d]) return fail(E_SHAPE, "einsum: extent of label %u differs", p[d]);
            }
            p += ranks[t];
        }
    }
    if (out->rank != n_out) return fail(E_RANK, "einsum: output rank %d, subscripts say %d", out->rank, n_out);
    for (int d = 0; d < n_out; ++d) {
        auto it = ext.find(ol[d]);
        if (it == ext.end()) return fail(E_ARG, "einsum: output label %u appears in no input", ol[d]);
        if (it->second != out->dims[d]) return fail(E_SHAPE, "einsum: output extent of label %u differs", ol[d]);
    }
    // free labels (distinct output labels) then summed labels; per-label stride into each tensor
    std::vector<uint32_t> free_l, sum_l;
    for (int d = 0; d < n_out; ++d)
        if (std::find(free_l.begin(), free_l.end(), ol[d]) == free_l.end()) free_l.push_back(ol[d]);
    for (auto& kv : ext)
        if (std::find(free_l.begin(), free_l.end(), kv.first) == free_l.end()) sum_l.push_back(kv.first);
    auto stride_in = [&](int t, uint32_t l) {
        const uint32_t* p = labels;
        for (int i = 0; i < t; ++i) p += ranks[i];
        int64_t s = 0;
        for (int d = 0; d < ranks[t]; ++d)
            if (p[d] == l) s += in[t].strides[d];  // repeated label = diagonal
        return s;
    };
    auto stride_out = [&](uint32_t l) {
        int64_t s = 0;
        for (int d = 0; d < n_out; ++d)
            if (ol[d] == l) s += out->strides[d];
        return s;
    };
    R* O = (R*)out->base + out->offset * NC;
    // 1. out = beta*out everywhere (zero where beta == 0): off-diagonal entries of a repeated
    //    output label receive no einsum contribution.
    {
        std::vector<Axis> ax;
        for (int d = 0; d < n_out; ++d) ax.push_back({ol[d], out->dims[d], {out->strides[d], 0, 0}});
        int64_t n = product(ax);
        for (int64_t i = 0; i < n; ++i) {
            R* dst = O + offset_of(ax, i, 0) * NC;
            if (be.is_zero()) {
                dst[0] = 0;
                if (CX) dst[1] = 0;
            } else {
                R dr = dst[0], di = CX ? dst[1] : R(0);
                dst[0] = be.re * dr - be.im * di;
                if (CX) dst[1] = be.re * di + be.im * dr;
            }
        }
    }
    // 2. out[free] += alpha * sum
    int nf = (int)free_l.size(), ns = (int)sum_l.size();
    std::vector<int64_t> fe(nf), se(ns), fo(nf);
    std::vector<std::vector<int64_t>> fs(n_in, std::vector<int64_t>(nf)), ss(n_in, std::vector<int64_t>(ns));
    for (int i = 0; i < nf; ++i) {
        fe[i] = ext[free_l[i]];
        fo[i] = stride_out(free_l[i]);
        for (int t = 0; t < n_in; ++t) fs[t][i] = stride_in(t, free_l[i]);
    }
    for (int i = 0; i < ns; ++i) {
        se[i] = ext[sum_l[i]];
        for (int t = 0; t < n_in; ++t) ss[t][i] = stride_in(t, sum_l[i]);
    }
    int64_t nfree = 1, nsum = 1;
    for (auto v : fe) nfree *= v;
    for (auto v : se) nsum *= v;
    std::vector<const R*> base(n_in);
    for (int t = 0; t < n_in; ++t) base[t] = (const R*)in[t].base + in[t].offset * NC;
    Sc<R, CX> one{R(1), R(0)};
    for (int64_t f = 0; f < nfree; ++f) {
        std::vector<int64_t> foff(n_in, 0);
        int64_t ooff = 0, lin = f;
        for (int i = nf - 1; i >= 0; --i) {
            int64_t idx = lin % fe[i];
            lin /= fe[i];
            ooff += idx * fo[i];
            for (int t = 0; t < n_in; ++t) foff[t] += idx * fs[t][i];
        }
        long double sr = 0, si = 0;
        for (int64_t s = 0; s < nsum; ++s) {
            long double pr = 1, pi = 0;
            for (int t = 0; t < n_in; ++t) {
                int64_t off = foff[t], l2 = s;
                for (int i = ns - 1; i >= 0; --i) {
                    off += (l2 % se[i]) * ss[t][i];
                    l2 /= se[i];
                }
                const R* x = base[t] + off * NC;
                if (CX) {
                    long double nr = pr * x[0] - pi * x[1], ni = pr * x[1] + pi * x[0];
                    pr = nr;
                    pi = ni;
                } else
                    pr *= x[0];
            }
            sr += pr;
            si += pi;
        }
        axpby<R, CX>(O + ooff * NC, al, (R)sr, (R)si, one);
    }
    return 0;
}

// ================================================================================================
// einsum along a pair list
// ================================================================================================
struct Node {
    std::vector<uint32_t> labels;
    tfo_view view;
    std::vector<char> storage;
};

template <class R, bool CX>
int einsum_pairs_impl(int dtype, int n_in, const tfo_view* in, const uint32_t* labels, const int32_t* ranks,
                      const uint32_t* ol, int n_out, const int32_t* pairs, int n_pairs, const void* alpha,
                      const void* beta, tfo_view* out) {
    constexpr int NC = CX ? 2 : 1;
    if (n_in < 2) return fail(E_ARG, "einsum_pairs: needs at least two operands");
    if (n_pairs != n_in - 1) return fail(E_ARG, "einsum_pairs: %d operands need %d pairs, got %d", n_in, n_in - 1, n_pairs);
    std::vector<Node> nodes((size_t)n_in);
    const uint32_t* p = labels;
    for (int t = 0; t < n_in; ++t) {
        nodes[t].labels.assign(p, p + ranks[t]);
        nodes[t].view = in[t];
        if (has_repeats(p, ranks[t])) return fail(E_ARG, "einsum_pairs: operand %d repeats a label", t);
        p += ranks[t];
    }
    std::vector<char> alive((size_t)n_in, 1);
    R one[2] = {1, 0}, zero[2] = {0, 0};
    for (int s = 0; s < n_pairs; ++s) {
        int i = pairs[2 * s], j = pairs[2 * s + 1];
        if (i < 0 || j < 0 || i >= (int)nodes.size() || j >= (int)nodes.size() || i == j || !alive[i] || !alive[j])
            return fail(E_ARG, "einsum_pairs: pair %d = (%d,%d) is not a valid contraction", s, i, j);
        alive[i] = alive[j] = 0;
        bool last = s == n_pairs - 1;
        Node nn;
        if (last) {
            nn.labels.assign(ol, ol + n_out);
        } else {
            // keep a label if the output or a surviving operand still needs it
            auto needed = [&](uint32_t l) {
                if (find_label(ol, n_out, l) >= 0) return true;
                for (size_t t = 0; t < nodes.size(); ++t)
                    if (alive[t] && find_label(nodes[t].labels.data(), (int)nodes[t].labels.size(), l) >= 0) return true;
                return false;
            };
            for (uint32_t l : nodes[i].labels)
                if (needed(l)) nn.labels.push_back(l);
            for (uint32_t l : nodes[j].labels)
                if (needed(l) && find_label(nn.labels.data(), (int)nn.labels.size(), l) < 0) nn.labels.push_back(l);
        }
        int rc;
        if (last) {
            rc = contract_impl<R, CX>(alpha, &nodes[i].view, nodes[i].labels.data(), &nodes[j].view,
                                      nodes[j].labels.data(), beta, out, ol);
        } else {
            tfo_view v{};
            v.rank = (int)nn.labels.size();
            int64_t n = 1;
            for (int d = v.rank - 1; d >= 0; --d) {
                uint32_t l = nn.labels[d];
                int ia = find_label(nodes[i].labels.data(), (int)nodes[i].labels.size(), l);
                v.dims[d] = ia >= 0 ? nodes[i].view.dims[ia]
                                    : nodes[j].view.dims[find_label(nodes[j].labels.data(), (int)nodes[j].labels.size(), l)];
                v.strides[d] = n;
                n *= v.dims[d];
            }
            nn.storage.resize((size_t)n * sizeof(R) * NC);
            v.base = nn.storage.data();
            nn.view = v;
            rc = contract_impl<R, CX>(one, &nodes[i].view, nodes[i].labels.data(), &nodes[j].view,
                                      nodes[j].labels.data(), zero, &nn.view, nn.labels.data());
        }
        if (rc) return rc;
        nodes[i].storage.clear();
        nodes[i].storage.shrink_to_fit();
        nodes[j].storage.clear();
        nodes[j].storage.shrink_to_fit();
        nodes.push_back(std::move(nn));
        nodes.back().view.base = last ? out->base : (void*)nodes.back().storage.data();
        alive.push_back(1);
    }
    (void)dtype;
    return 0;
}

// ---- diagonal helpers for Trace / AntiTrace / AntiDiag --------------------------------------------
// Collapses each pair (i, j) of `modes` on view v into the single label i whose stride is the sum
// of both strides (a zero-copy diagonal, tenferro-tensor/src/lib.rs:518-529).
int take_diagonal(tfo_view& v, std::vector<uint32_t>& modes, const uint32_t* pairs, int n_pairs) {
    for (int p = 0; p < n_pairs; ++p) {
        uint32_t li = pairs[2 * p], lj = pairs[2 * p + 1];
        int i = find_label(modes.data(), (int)modes.size(), li), j = find_label(modes.data(), (int)modes.size(), lj);
        if (i < 0 || j < 0 || i == j) return fail(E_ARG, "paired modes (%u,%u) must both label distinct axes", li, lj);
        if (v.dims[i] != v.dims[j]) return fail(E_SHAPE, "paired modes (%u,%u) have different extents", li, lj);
        v.strides[i] += v.strides[j];
        for (int d = j; d + 1 < v.rank; ++d) {
            v.dims[d] = v.dims[d + 1];
            v.strides[d] = v.strides[d + 1];
        }
        modes.erase(modes.begin() + j);
        v.rank--;
    }
    return 0;
}

template <class R, bool CX>
int scale_all(const void* beta, tfo_view* c) {
    constexpr int NC = CX ? 2 : 1;
    auto be = Sc<R, CX>::load(beta);
    std::vector<Axis> ax;
    for (int d = 0; d < c->rank; ++d) ax.push_back({0u, c->dims[d], {c->strides[d], 0, 0}});
    R* C = (R*)c->base + c->offset * NC;
    int64_t n = product(ax);
    Sc<R, CX> zero{0, 0};
    for (int64_t i = 0; i < n; ++i) axpby<R, CX>(C + offset_of(ax, i, 0) * NC, zero, 0, 0, be);
    return 0;
}

#define DISPATCH(dt, fn, ...)                                                        \
    switch (dt) {                                                                    \
        case TFO_F32: return fn<float, false>(__VA_ARGS__);                          \
        case TFO_F64: return fn<double, false>(__VA_ARGS__);                         \
        case TFO_C64: return fn<float, true>(__VA_ARGS__);                           \
        case TFO_C128: return fn<double, true>(__VA_ARGS__);                         \
        default: return fail(E_ARG, "unknown dtype %d", dt);                         \
    }

}  // namespace

extern "C" {

const char* tfo_last_message(void) { return g_msg.c_str(); }
int tfo_num_threads(void) { return nthreads(); }
void tfo_set_num_threads(int n) { g_threads = n; }

int tfo_permute(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const void* beta,
                tfo_view* b, const uint32_t* modes_b) {
    if (a->rank != b->rank) return fail(E_RANK, "permute: rank %d vs %d", a->rank, b->rank);
    if (has_repeats(modes_a, a->rank) || has_repeats(modes_b, b->rank)) return fail(E_ARG, "permute: repeated mode label");
    DISPATCH(dtype, permute_impl, alpha, a, modes_a, beta, b, modes_b)
}
int tfo_reduce(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const void* beta,
               tfo_view* c, const uint32_t* modes_c, int op) {
    DISPATCH(dtype, reduce_impl, alpha, a, modes_a, beta, c, modes_c, op)
}
int tfo_contract(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const tfo_view* b,
                 const uint32_t* modes_b, const void* beta, tfo_view* c, const uint32_t* modes_c) {
    DISPATCH(dtype, contract_impl, alpha, a, modes_a, b, modes_b, beta, c, modes_c)
}
int tfo_contract_naive(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const tfo_view* b,
                       const uint32_t* modes_b, const void* beta, tfo_view* c, const uint32_t* modes_c) {
    DISPATCH(dtype, contract_naive_impl, alpha, a, modes_a, b, modes_b, beta, c, modes_c)
}
int tfo_batched_gemm(int dtype, int n_batch, const void* alpha, const tfo_view* a, const tfo_view* b,
                     const void* beta, tfo_view* c) {
    // C[batch,m,n] = alpha*A[batch,m,k]*B[batch,k,n] + beta*C: labels 0..nb-1 batch, then m, n, k
    if (a->rank != n_batch + 2 || b->rank != n_batch + 2 || c->rank != n_batch + 2)
        return fail(E_RANK, "batched_gemm: every view must have rank n_batch+2 = %d", n_batch + 2);
    std::vector<uint32_t> ma, mb, mc;
    for (int i = 0; i < n_batch; ++i) {
        ma.push_back(i);
        mb.push_back(i);
        mc.push_back(i);
    }
    uint32_t m = n_batch, n = n_batch + 1, k = n_batch + 2;
    ma.push_back(m); ma.push_back(k);
    mb.push_back(k); mb.push_back(n);
    mc.push_back(m); mc.push_back(n);
    return tfo_contract(dtype, alpha, a, ma.data(), b, mb.data(), beta, c, mc.data());
}
int tfo_elementwise_mul(int dtype, const void* alpha, const tfo_view* a, const tfo_view* b, const void* beta,
                        tfo_view* c) {
    DISPATCH(dtype, emul_impl, alpha, a, b, beta, c)
}
int tfo_conj(int dtype, const tfo_view* in, tfo_view* out) { DISPATCH(dtype, conj_impl, in, out) }

int tfo_trace(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const void* beta,
              tfo_view* c, const uint32_t* modes_c, const uint32_t* pairs, int n_pairs) {
    // sum over the diagonal of every pair = Reduce of the diagonal view with the pair label dropped
    tfo_view d = *a;
    std::vector<uint32_t> m(modes_a, modes_a + a->rank);
    if (int e = take_diagonal(d, m, pairs, n_pairs)) return e;
    for (int p = 0; p < n_pairs; ++p)
        if (find_label(modes_c, c->rank, pairs[2 * p]) >= 0 || find_label(modes_c, c->rank, pairs[2 * p + 1]) >= 0)
            return fail(E_ARG, "trace: paired mode appears in the output");
    return tfo_reduce(dtype, alpha, &d, m.data(), beta, c, modes_c, TFO_SUM);
}
static int anti_common(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const void* beta,
                       tfo_view* c, const uint32_t* modes_c, const uint32_t* pairs, int n_pairs, bool a_has_i) {
    // 1. C = beta*C everywhere; 2. diagonal(C) += alpha * A (broadcast over the pair label if A lacks it)
    int rc;
    switch (dtype) {
        case TFO_F32: rc = scale_all<float, false>(beta, c); break;
        case TFO_F64: rc = scale_all<double, false>(beta, c); break;
        case TFO_C64: rc = scale_all<float, true>(beta, c); break;
        case TFO_C128: rc = scale_all<double, true>(beta, c); break;
        default: return fail(E_ARG, "unknown dtype %d", dtype);
    }
    if (rc) return rc;
    tfo_view d = *c;
    std::vector<uint32_t> mc(modes_c, modes_c + c->rank);
    if (int e = take_diagonal(d, mc, pairs, n_pairs)) return e;
    // input view aligned to the diagonal view's modes; stride 0 where A does not carry the label
    tfo_view av{};
    av.base = a->base;
    av.offset = a->offset;
    av.rank = d.rank;
    for (int x = 0; x < d.rank; ++x) {
        int j = find_label(modes_a, a->rank, mc[x]);
        av.dims[x] = d.dims[x];
        if (j >= 0) {
            if (a->dims[j] != d.dims[x]) return fail(E_SHAPE, "anti: extent of mode %u differs", mc[x]);
            av.strides[x] = a->strides[j];
        } else {
            bool is_pair_label = false;
            for (int p = 0; p < n_pairs; ++p) is_pair_label |= pairs[2 * p] == mc[x];
            if (!is_pair_label || a_has_i) return fail(E_ARG, "anti: output mode %u missing from the input", mc[x]);
            av.strides[x] = 0;
        }
    }
    double one[2] = {1, 0};
    float onef[2] = {1, 0};
    const void* o = (dtype == TFO_F32 || dtype == TFO_C64) ? (const void*)onef : (const void*)one;
    return tfo_permute(dtype, alpha, &av, mc.data(), o, &d, mc.data());
}
int tfo_anti_trace(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const void* beta,
                   tfo_view* c, const uint32_t* modes_c, const uint32_t* pairs, int n_pairs) {
    return anti_common(dtype, alpha, a, modes_a, beta, c, modes_c, pairs, n_pairs, false);
}
int tfo_anti_diag(int dtype, const void* alpha, const tfo_view* a, const uint32_t* modes_a, const void* beta,
                  tfo_view* c, const uint32_t* modes_c, const uint32_t* pairs, int n_pairs) {
    return anti_common(dtype, alpha, a, modes_a, beta, c, modes_c, pairs, n_pairs, true);
}

int tfo_einsum_naive(int dtype, int n_inputs, const tfo_view* inputs, const uint32_t* labels, const int32_t* ranks,
                     const uint32_t* out_labels, int n_out, const void* alpha, const void* beta, tfo_view* out) {
    DISPATCH(dtype, einsum_naive_impl, n_inputs, inputs, labels, ranks, out_labels, n_out, alpha, beta, out)
}
int tfo_einsum_pairs(int dtype, int n_inputs, const tfo_view* inputs, const uint32_t* labels, const int32_t* ranks,
                     const uint32_t* out_labels, int n_out, const int32_t* pairs, int n_pairs, const void* alpha,
                     const void* beta, tfo_view* out) {
    DISPATCH(dtype, einsum_pairs_impl, dtype, n_inputs, inputs, labels, ranks, out_labels, n_out, pairs, n_pairs,
             alpha, beta, out)
}

}  // extern "C"
