// host_backend.cpp -- stand-ins for the device launchers, over HOST memory, for the sanitizer build of the backend's host
// code (tests/cpp/test_host_sanitized.cpp).
//
// The host side of the library -- descriptor validation and plans (plan.cpp), the dispatch of every operation onto
// copy / reduce / contract launches (prims.cpp), the einsum parser, tree optimiser and executor (einsum.cpp) and the error
// records (errors.cpp) -- is compiled unchanged with AddressSanitizer and UndefinedBehaviorSanitizer and linked against
// the functions below instead of the HIP launchers.  Each one has the signature and the meaning of the launcher it
// stands in for (tenferro-rs_amd/csrc/internal.hpp) and computes it with one plain loop nest in complex double
// arithmetic, so a whole call -- views in, result out -- runs on the CPU with every host-side index, stride table and
// buffer lifetime under the sanitizers, and its result can be compared with the oracle's.
// Test infrastructure only: nothing here is linked into libtenferro_hip.so.
#include <atomic>
#include <complex>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <set>

#include "../../tenferro-rs_amd/csrc/internal.hpp"

namespace tfh {
namespace {
using cd = std::complex<double>;

cd load(int dt, const void* base, int64_t at) {
    switch (dt) {
        case TFH_F32: return cd(((const float*)base)[at], 0.0);
        case TFH_F64: return cd(((const double*)base)[at], 0.0);
        case TFH_C64: return cd(((const float*)base)[2 * at], ((const float*)base)[2 * at + 1]);
        default: return cd(((const double*)base)[2 * at], ((const double*)base)[2 * at + 1]);
    }
}

void store(int dt, void* base, int64_t at, cd v) {
    switch (dt) {
        case TFH_F32: ((float*)base)[at] = (float)v.real(); break;
        case TFH_F64: ((double*)base)[at] = v.real(); break;
        case TFH_C64:
            ((float*)base)[2 * at] = (float)v.real();
            ((float*)base)[2 * at + 1] = (float)v.imag();
            break;
        default:
            ((double*)base)[2 * at] = v.real();
            ((double*)base)[2 * at + 1] = v.imag();
    }
}

// Visits every index of `axes`, handing the element offset in each of the three slots to `f`.
void walk(const std::vector<Axis>& axes, const std::function<void(int64_t, int64_t, int64_t)>& f) {
    for (const Axis& x : axes)
        if (x.n <= 0) return;
    std::vector<int64_t> idx(axes.size(), 0);
    int64_t o[3] = {0, 0, 0};
    for (;;) {
        f(o[0], o[1], o[2]);
        int d = (int)axes.size() - 1;
        for (; d >= 0; --d) {
            for (int s = 0; s < 3; ++s) o[s] += axes[d].s[s];
            if (++idx[d] < axes[d].n) break;
            for (int s = 0; s < 3; ++s) o[s] -= axes[d].s[s] * axes[d].n;
            idx[d] = 0;
        }
        if (d < 0) return;
    }
}

cd scale(Scalar s) { return cd(s.re, s.im); }

// beta == 0 overwrites without reading the output (tenferro-prims/src/lib.rs:300-304)
cd combine(int dt, Scalar alpha, cd value, Scalar beta, const void* out, int64_t at) {
    cd r = scale(alpha) * value;
    if (!beta.is_zero()) r += scale(beta) * load(dt, out, at);
    return r;
}

std::mutex g_mu;
std::set<void*> g_live;   // blocks handed out by pool_alloc and not yet given back
}  // namespace

int32_t launch_copy(int dtype, const void* in, void* out, std::vector<Axis> axes, Scalar alpha, Scalar beta, bool conj, void*) {
    walk(axes, [&](int64_t i, int64_t o, int64_t) {
        cd v = load(dtype, in, i);
        if (conj) v = std::conj(v);
        store(dtype, out, o, combine(dtype, alpha, v, beta, out, o));
    });
    return TFH_OK;
}

int32_t launch_fill(int dtype, void* out, std::vector<Axis> axes, Scalar value, void*) {
    walk(axes, [&](int64_t o, int64_t, int64_t) { store(dtype, out, o, scale(value)); });
    return TFH_OK;
}

int32_t launch_emul(int dtype, const void* a, const void* b, void* c, std::vector<Axis> axes, Scalar alpha, Scalar beta, void*) {
    walk(axes, [&](int64_t ia, int64_t ib, int64_t ic) {
        store(dtype, c, ic, combine(dtype, alpha, load(dtype, a, ia) * load(dtype, b, ib), beta, c, ic));
    });
    return TFH_OK;
}

int32_t launch_reduce(int dtype, const void* a, void* c, std::vector<Axis> kept, std::vector<Axis> red, int reduce_op, Scalar alpha,
                      Scalar beta, void*) {
    if (reduce_op != TFH_REDUCE_SUM && is_complex(dtype)) return set_error(TFH_ERR_INVALID_ARGUMENT, "Max/Min of a complex tensor");
    walk(kept, [&](int64_t ia, int64_t ic, int64_t) {
        cd acc(0.0, 0.0);
        bool first = true;
        walk(red, [&](int64_t ir, int64_t, int64_t) {
            const cd v = load(dtype, a, ia + ir);
            if (reduce_op == TFH_REDUCE_SUM) acc += v;
            else if (first) acc = v;
            else if (reduce_op == TFH_REDUCE_MAX) acc = cd(std::max(acc.real(), v.real()), 0.0);
            else acc = cd(std::min(acc.real(), v.real()), 0.0);
            first = false;
        });
        store(dtype, c, ic, combine(dtype, alpha, acc, beta, c, ic));
    });
    return TFH_OK;
}

// The stand-in's routed launch: the classified axes.  A repeated call with the same strides (contract_cache.cpp) runs the
// loop nest over them again on the new buffers.
namespace {
struct HostRecord : ContractRecord {
    ContractAxes ax;
    int conj = 0;
};
std::atomic<int64_t> g_replays{0};
}  // namespace
int64_t host_backend_replays() { return g_replays.load(); }

int32_t launch_contract(int dtype, const void* a, const void* b, void* c, ContractAxes ax, Scalar alpha, Scalar beta, void*, int conj,
                        std::shared_ptr<ContractRecord>* record) {
    if (record) {
        auto r = std::make_shared<HostRecord>();
        r->ax = ax;
        r->conj = conj;
        r->label = "(host loop nest)";
        *record = std::move(r);
    }
    std::vector<Axis> free_axes = ax.batch;
    free_axes.insert(free_axes.end(), ax.M.begin(), ax.M.end());
    free_axes.insert(free_axes.end(), ax.N.begin(), ax.N.end());
    walk(free_axes, [&](int64_t ia, int64_t ib, int64_t ic) {
        cd acc(0.0, 0.0);
        walk(ax.K, [&](int64_t ka, int64_t kb, int64_t) {
            cd x = load(dtype, a, ia + ka), y = load(dtype, b, ib + kb);
            if (conj & 1) x = std::conj(x);
            if (conj & 2) y = std::conj(y);
            acc += x * y;
        });
        store(dtype, c, ic, combine(dtype, alpha, acc, beta, c, ic));
    });
    return TFH_OK;
}

bool replay_contract(const ContractRecord& rec, int dtype, const void* a, const void* b, void* c, Scalar alpha, Scalar beta, void* stream,
                     int32_t& status) {
    const HostRecord& r = static_cast<const HostRecord&>(rec);
    ++g_replays;
    status = launch_contract(dtype, a, b, c, r.ax, alpha, beta, stream, r.conj, nullptr);
    return true;
}

// Grouped plans keep device tables; they are outside what the sanitizer build covers.
int32_t grouped_plan_init(tfh_plan&) { return set_error(TFH_ERR_DEVICE, "grouped plans need a device"); }
int32_t launch_grouped(const tfh_plan&, Scalar, const tfh_view*, Scalar, tfh_view*, void*) {
    return set_error(TFH_ERR_DEVICE, "grouped plans need a device");
}
void grouped_state_destroy(GroupedState*) {}

// Every intermediate is its own heap block of exactly the size asked for, so an access past either end of it is an
// AddressSanitizer report, and a block that is never given back is a leak report at exit.
int32_t pool_alloc(void*, size_t bytes, void** out) {
    *out = std::malloc(bytes ? bytes : 1);
    if (!*out) return set_error(TFH_ERR_DEVICE, "out of memory");
    std::lock_guard<std::mutex> lk(g_mu);
    g_live.insert(*out);
    return TFH_OK;
}

void pool_free(void*, void* ptr) {
    if (!ptr) return;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (!g_live.erase(ptr)) {
            std::fprintf(stderr, "pool_free of a block that pool_alloc did not hand out (or a second free)\n");
            std::abort();
        }
    }
    std::free(ptr);
}

size_t host_backend_live_blocks() {
    std::lock_guard<std::mutex> lk(g_mu);
    return g_live.size();
}
}  // namespace tfh
