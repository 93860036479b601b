// test_host_sanitized.cpp -- the host code of the backend and the oracle under AddressSanitizer + UndefinedBehaviorSanitizer.
//
// Linked from: tenferro-rs_amd/csrc/{errors,plan,prims,einsum,contract_cache}.cpp (unchanged), tests/cpp/host_backend.cpp (stand-ins for the
// device launchers over host memory) and oracle/tfo_oracle.cpp, all compiled with -fsanitize=address,undefined.  Every
// operand and result is a heap block of exactly its size, so an index or stride mistake anywhere between the C entry point
// and the innermost loop is a sanitizer report; results are compared with the oracle's, which is itself checked here
// against its brute-force form at sizes that span several cache blocks and all its threads.
//
//   ./test_host_sanitized        prints "<n> checks, 0 failed" and exits 0, or the first failures and exits 1
#include <algorithm>
#include <cmath>
#include <complex>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/tenferro_hip.h"
#include "../../oracle/tfo_oracle.h"

namespace tfh {
size_t host_backend_live_blocks();
int64_t host_backend_replays();   // contractions that ran from a routed launch kept in a plan (host_backend.cpp)
int32_t set_no_compatible_device(int32_t space_kind, int64_t space_id, int32_t op_kind);   // errors.cpp
}

static int g_checks = 0, g_failed = 0;
#define CHECK(cond)                                                                       \
    do {                                                                                  \
        ++g_checks;                                                                       \
        if (!(cond)) {                                                                    \
            if (++g_failed <= 20) std::printf("FAILED %s:%d  %s\n", __FILE__, __LINE__, #cond); \
        }                                                                                 \
    } while (0)

struct Rng {   // xorshift64*: the same sequence on every run
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 2654435761u + 88172645463325252ull) {}
    uint64_t next() { s ^= s >> 12; s ^= s << 25; s ^= s >> 27; return s * 2685821657736338717ull; }
    int below(int n) { return (int)(next() % (uint64_t)n); }
    double uniform() { return (double)(next() >> 11) / 9007199254740992.0 * 2.0 - 1.0; }
};

static size_t elem_size(int dt) { return dt == TFH_F32 ? 4 : dt == TFH_C128 ? 16 : 8; }
static bool is_cx(int dt) { return dt == TFH_C64 || dt == TFH_C128; }
static double tol_of(int dt) { return (dt == TFH_F32 || dt == TFH_C64) ? 1e-5 : 1e-12; }

// A tensor on the heap with an arbitrary (possibly permuted, reversed or broadcast) layout; the block holds exactly the
// elements the view can reach.
struct HostTensor {
    int dt = TFH_F64;
    std::vector<int64_t> dims, strides;
    int64_t offset = 0, span = 1;
    void* data = nullptr;
    HostTensor() = default;
    HostTensor(const HostTensor&) = delete;
    HostTensor& operator=(const HostTensor&) = delete;
    ~HostTensor() { std::free(data); }

    // layout: 0 = row-major, 1 = column-major, 2 = random axis order, 3 = random order with one axis reversed,
    // 4 = random order with one axis broadcast (stride 0; inputs only)
    void init(int dtype, const std::vector<int64_t>& d, int layout, Rng& rng) {
        dt = dtype;
        dims = d;
        const int r = (int)d.size();
        strides.assign(r, 0);
        std::vector<int> order(r);
        for (int i = 0; i < r; ++i) order[i] = layout == 1 ? i : r - 1 - i;   // fastest axis first
        if (layout >= 2)
            for (int i = r - 1; i > 0; --i) std::swap(order[i], order[rng.below(i + 1)]);
        const int special = r ? rng.below(r) : -1;
        int64_t run = 1;
        for (int i = 0; i < r; ++i) {
            const int axis = order[i];
            if (layout == 4 && axis == special) continue;   // stride stays 0
            strides[axis] = run;
            run *= std::max<int64_t>(d[axis], 1);
        }
        span = run;
        offset = 0;
        if (layout == 3 && r && d[special] > 1) {
            offset = strides[special] * (d[special] - 1);
            strides[special] = -strides[special];
        }
        data = std::malloc((size_t)span * elem_size(dt));
        const int n = (int)span * (is_cx(dt) ? 2 : 1);
        for (int i = 0; i < n; ++i) {
            if (dt == TFH_F32 || dt == TFH_C64) ((float*)data)[i] = (float)rng.uniform();
            else ((double*)data)[i] = rng.uniform();
        }
    }
    int64_t count() const { int64_t n = 1; for (int64_t x : dims) n *= x; return n; }
    void view_into(void* out) const {   // tfh_view and tfo_view share one layout
        tfh_view v;
        std::memset(&v, 0, sizeof v);
        v.base = data;
        v.rank = (int32_t)dims.size();
        v.offset = offset;
        for (size_t i = 0; i < dims.size(); ++i) { v.dims[i] = dims[i]; v.strides[i] = strides[i]; }
        std::memcpy(out, &v, sizeof v);
    }
    tfh_view view() const { tfh_view v; view_into(&v); return v; }
    tfo_view oview() const { static_assert(sizeof(tfo_view) == sizeof(tfh_view), "views share a layout"); tfo_view v; view_into(&v); return v; }
    void copy_data_from(const HostTensor& o) { std::memcpy(data, o.data, (size_t)span * elem_size(dt)); }
    void conj_clone_of(const HostTensor& o) {   // same layout, every element conjugated
        dt = o.dt; dims = o.dims; strides = o.strides; offset = o.offset; span = o.span;
        data = std::malloc((size_t)span * elem_size(dt));
        copy_data_from(o);
        if (!is_cx(dt)) return;
        for (int64_t i = 0; i < span; ++i) {
            if (dt == TFH_C64) ((float*)data)[2 * i + 1] = -((float*)data)[2 * i + 1];
            else ((double*)data)[2 * i + 1] = -((double*)data)[2 * i + 1];
        }
    }
    std::complex<double> at(const std::vector<int64_t>& idx) const {
        int64_t e = offset;
        for (size_t i = 0; i < dims.size(); ++i) e += idx[i] * strides[i];
        if (dt == TFH_F32) return ((float*)data)[e];
        if (dt == TFH_F64) return ((double*)data)[e];
        if (dt == TFH_C64) return {((float*)data)[2 * e], ((float*)data)[2 * e + 1]};
        return {((double*)data)[2 * e], ((double*)data)[2 * e + 1]};
    }
};

// relative Frobenius distance of two tensors of the same dims (any layouts)
static double rel_err(const HostTensor& x, const HostTensor& ref) {
    std::vector<int64_t> idx(x.dims.size(), 0);
    double num = 0, den = 0;
    if (x.count() == 0) return 0;
    for (;;) {
        const auto a = x.at(idx), b = ref.at(idx);
        num += std::norm(a - b);
        den += std::norm(b);
        int d = (int)idx.size() - 1;
        for (; d >= 0; --d) {
            if (++idx[d] < x.dims[d]) break;
            idx[d] = 0;
        }
        if (d < 0) break;
    }
    return std::sqrt(num) / std::max(std::sqrt(den), 1e-300);
}

struct ScalarBytes { double v[2]; float f[2]; const void* ptr(int dt) const { return (dt == TFH_F32 || dt == TFH_C64) ? (const void*)f : (const void*)v; } };
static ScalarBytes scalar(int dt, double re, double im) {
    ScalarBytes s;
    s.v[0] = re; s.v[1] = is_cx(dt) ? im : 0.0;
    s.f[0] = (float)re; s.f[1] = is_cx(dt) ? (float)im : 0.0f;
    return s;
}

// ------------------------------------------------------------------------------------------------ errors
static void error_records() {
    tfh_error_info info;
    // the record tfh_preferred_compute_devices leaves for a memory space this library does not compute on
    CHECK(tfh::set_no_compatible_device(TFH_SPACE_MAIN_MEMORY, 0, TFH_KIND_PERMUTE) == TFH_ERR_NO_COMPATIBLE_DEVICE);
    tfh_last_error(&info);
    CHECK(info.status == TFH_ERR_NO_COMPATIBLE_DEVICE && info.n_expected == 2 && info.expected[0] == TFH_SPACE_MAIN_MEMORY);
    CHECK(info.n_got == 1 && info.got[0] == TFH_KIND_PERMUTE);
    CHECK(std::string(info.message) == "no compatible compute device for Permute on MainMemory");
    // a shape mismatch at the maximum rank with extents whose decimal form overflows the formatting buffers
    std::vector<int64_t> big(TFH_MAX_RANK, INT64_MAX / 3), other(TFH_MAX_RANK, INT64_MAX / 5);
    uint32_t modes[TFH_MAX_RANK];
    for (int i = 0; i < TFH_MAX_RANK; ++i) modes[i] = (uint32_t)i;
    tfh_desc d;
    std::memset(&d, 0, sizeof d);
    d.op = TFH_OP_PERMUTE;
    d.modes_a = modes; d.n_modes_a = TFH_MAX_RANK;
    d.modes_c = modes; d.n_modes_c = TFH_MAX_RANK;
    const int64_t* shapes[2] = {big.data(), other.data()};
    int32_t ranks[2] = {TFH_MAX_RANK, TFH_MAX_RANK};
    tfh_plan* p = nullptr;
    const int32_t st = tfh_plan_create(TFH_F64, &d, shapes, ranks, 2, &p);
    CHECK(st == TFH_ERR_SHAPE_MISMATCH && p == nullptr);
    tfh_last_error(&info);
    CHECK(info.n_expected == TFH_MAX_RANK && info.n_got == TFH_MAX_RANK && std::strlen(info.message) < sizeof info.message);
    // a notation far longer than the message buffer
    std::string longn(5000, '(');
    tfh_subscripts* s = nullptr;
    CHECK(tfh_subscripts_parse(longn.c_str(), &s) == TFH_ERR_INVALID_ARGUMENT && s == nullptr);
    tfh_last_error(&info);
    CHECK(std::strlen(info.message) < sizeof info.message);
    for (int st_ = -2; st_ < 12; ++st_) CHECK(tfh_status_name(st_) != nullptr);
    CHECK(tfh_dtype_size(TFH_C128) == 16 && tfh_dtype_size(99) == 0);
}

// ------------------------------------------------------------------------------------------------ parser
static void parser_cases(Rng& rng) {
    const char* good[] = {"ij,jk->ik", "ij,(jk,kl)->il", "((ab,bc),cd),de->ae", "i->", "->", "ii->i", "i->ii", "ab,ab->", "a,b->ab",
                          "ijk->kji", " ij , jk -> ik ", "aB,Bc->ac", "(ij,jk),(kl,lm)->im"};
    for (const char* g : good) {
        tfh_subscripts* s = nullptr;
        CHECK(tfh_subscripts_parse(g, &s) == TFH_OK && s != nullptr);
        if (!s) continue;
        const int n = tfh_subscripts_n_inputs(s);
        uint32_t lab[1];
        for (int i = -1; i <= n; ++i) tfh_subscripts_labels(s, i, lab, 1);      // capacity smaller than most ranks
        for (int i = -2; i <= n + 1; ++i) tfh_subscripts_input_rank(s, i);
        char small[4];
        tfh_subscripts_nesting(s, small, sizeof small);
        char buf[256];
        CHECK(tfh_subscripts_nesting(s, buf, sizeof buf) >= 0);
        tfh_subscripts_destroy(s);
    }
    const char* bad[] = {"ij,jk", "ij->k", "(ij,jk->ik", "ij,jk)->ik", "i j->", "ij,,jk->ik", "ij->->i", "1j->j", "ij,jk->ikz", "(),a->a",
                         "(ij),jk->ik", "ij,(jk)->ik", "a->a->a", ",->", "(a,b,c)->abc"};
    for (const char* b : bad) {
        tfh_subscripts* s = nullptr;
        const int32_t st = tfh_subscripts_parse(b, &s);
        CHECK((st == TFH_OK) == (s != nullptr));   // some of these are legal in a lenient grammar; none may crash or leak
        if (s) tfh_subscripts_destroy(s);
    }
    CHECK(tfh_subscripts_parse(nullptr, nullptr) != TFH_OK);
    // random strings over the grammar's alphabet: every one parses or is refused, and what parses can be optimised
    const char alphabet[] = "abcdij,,()->- Z";
    for (int iter = 0; iter < 20000; ++iter) {
        std::string t;
        const int len = rng.below(14);
        for (int i = 0; i < len; ++i) t.push_back(alphabet[rng.below((int)sizeof alphabet - 1)]);
        tfh_subscripts* s = nullptr;
        const int32_t st = tfh_subscripts_parse(t.c_str(), &s);
        ++g_checks;
        if ((st == TFH_OK) != (s != nullptr)) { ++g_failed; std::printf("FAILED parse '%s'\n", t.c_str()); }
        if (!s) continue;
        const int n = tfh_subscripts_n_inputs(s);
        std::vector<std::vector<int64_t>> dims(n);
        std::vector<const int64_t*> ptrs(n);
        std::vector<int32_t> ranks(n);
        for (int i = 0; i < n; ++i) {
            ranks[i] = tfh_subscripts_input_rank(s, i);
            dims[i].assign(std::max(ranks[i], 1), 2);
            ptrs[i] = dims[i].data();
        }
        tfh_tree* tree = nullptr;
        if (tfh_tree_optimize(s, ptrs.data(), ranks.data(), n, &tree) == TFH_OK && tree) {
            uint32_t lab[2]; int64_t dm[2];
            for (int node = -1; node < n + tfh_tree_n_steps(tree) + 1; ++node) tfh_tree_node(tree, node, lab, dm, 2);
            int64_t od[1];
            tfh_tree_output_dims(tree, od, 1);
            tfh_tree_destroy(tree);
        }
        tfh_subscripts_destroy(s);
    }
}

// ------------------------------------------------------------------------------------------------ plans
static void plan_validation(Rng& rng) {
    // random descriptors against random shapes: every one is accepted or refused with a status, none may read past the
    // arrays it was given
    for (int iter = 0; iter < 20000; ++iter) {
        tfh_desc d;
        std::memset(&d, 0, sizeof d);
        d.op = rng.below(10) - 1;
        d.reduce_op = rng.below(4);
        std::vector<uint32_t> ma(rng.below(5)), mb(rng.below(5)), mc(rng.below(5)), pairs(2 * rng.below(3));
        for (auto& x : ma) x = (uint32_t)rng.below(5);
        for (auto& x : mb) x = (uint32_t)rng.below(5);
        for (auto& x : mc) x = (uint32_t)rng.below(5);
        for (auto& x : pairs) x = (uint32_t)rng.below(5);
        std::vector<int64_t> batch(rng.below(3));
        for (auto& x : batch) x = rng.below(4);
        d.batch_dims = batch.data(); d.n_batch_dims = (int32_t)batch.size();
        d.m = rng.below(4); d.n = rng.below(4); d.k = rng.below(4);
        d.modes_a = ma.data(); d.n_modes_a = (int32_t)ma.size();
        d.modes_b = mb.data(); d.n_modes_b = (int32_t)mb.size();
        d.modes_c = mc.data(); d.n_modes_c = (int32_t)mc.size();
        d.paired = pairs.data(); d.n_pairs = (int32_t)pairs.size() / 2;
        const int nt = rng.below(4) + 1;
        std::vector<std::vector<int64_t>> shp(nt);
        std::vector<const int64_t*> ptrs(nt);
        std::vector<int32_t> ranks(nt);
        for (int t = 0; t < nt; ++t) {
            shp[t].resize(rng.below(5));
            for (auto& x : shp[t]) x = rng.below(4);
            if (shp[t].empty()) shp[t].reserve(1);
            ptrs[t] = shp[t].data();
            ranks[t] = (int32_t)shp[t].size();
        }
        tfh_plan* p = nullptr;
        const int32_t st = tfh_plan_create(rng.below(6) - 1, &d, ptrs.data(), ranks.data(), nt, &p);
        ++g_checks;
        if ((st == TFH_OK) != (p != nullptr)) { ++g_failed; std::printf("FAILED plan fuzz %d\n", iter); }
        if (p) {
            char buf[8];
            tfh_plan_describe(p, buf, sizeof buf);
            tfh_plan_destroy(p);
        }
    }
}

// ------------------------------------------------------------------------------------------------ primitives vs the oracle
struct Labels { std::vector<uint32_t> v; };

static void prims_against_oracle(Rng& rng) {
    for (int iter = 0; iter < 400; ++iter) {
        const int dt = rng.below(4);
        const int64_t ext[6] = {1 + rng.below(5), 1 + rng.below(5), 1 + rng.below(4), 1 + rng.below(4), 1 + rng.below(3), 1 + rng.below(3)};
        auto dims_of = [&](const std::vector<uint32_t>& m) { std::vector<int64_t> d; for (uint32_t l : m) d.push_back(ext[l]); return d; };
        auto shuffled = [&](int n) { std::vector<uint32_t> m(n); for (int i = 0; i < n; ++i) m[i] = (uint32_t)i; for (int i = n - 1; i > 0; --i) std::swap(m[i], m[rng.below(i + 1)]); return m; };
        const ScalarBytes alpha = scalar(dt, 0.5 + rng.uniform(), rng.uniform()), beta = rng.below(3) ? scalar(dt, rng.uniform(), rng.uniform()) : scalar(dt, 0, 0);
        tfh_desc d;
        std::memset(&d, 0, sizeof d);
        const int kind = rng.below(5);
        std::vector<uint32_t> ma, mb, mc;
        if (kind == 0) {   // Permute
            const int r = rng.below(5);
            ma = shuffled(r); mc = shuffled(r);
            d.op = TFH_OP_PERMUTE;
        } else if (kind == 1) {   // Reduce
            const int r = 1 + rng.below(4);
            ma = shuffled(r);
            for (uint32_t l : shuffled(r)) if (rng.below(2)) mc.push_back(l);
            d.op = TFH_OP_REDUCE;
            d.reduce_op = is_cx(dt) ? TFH_REDUCE_SUM : rng.below(3);
        } else if (kind == 2) {   // Contract: every label in two of the three tensors, or in all three (batch)
            for (uint32_t l = 0; l < 6; ++l) {
                const int where = rng.below(5);   // 0 skip, 1 M, 2 N, 3 K, 4 batch
                if (where == 1 || where == 3 || where == 4) ma.push_back(l);
                if (where == 2 || where == 3 || where == 4) mb.push_back(l);
                if (where == 1 || where == 2 || where == 4) mc.push_back(l);
            }
            for (auto* m : {&ma, &mb, &mc}) for (int i = (int)m->size() - 1; i > 0; --i) std::swap((*m)[i], (*m)[rng.below(i + 1)]);
            d.op = TFH_OP_CONTRACT;
        } else if (kind == 3) {   // ElementwiseMul
            const int r = rng.below(4);
            ma = mb = mc = shuffled(r);
            d.op = TFH_OP_ELEMENTWISE_MUL;
        } else {   // Trace over one pair of equal extents
            ma = {0, 1, 2}; mc = {2};
            d.op = TFH_OP_TRACE;
        }
        int64_t ext_local[6];
        std::memcpy(ext_local, ext, sizeof ext);
        std::vector<int64_t> da = dims_of(ma), db = dims_of(mb), dc = dims_of(mc);
        uint32_t pair01[2] = {0, 1};
        if (kind == 4) { da[1] = da[0]; d.paired = pair01; d.n_pairs = 1; }
        d.modes_a = ma.data(); d.n_modes_a = (int32_t)ma.size();
        d.modes_b = mb.data(); d.n_modes_b = (int32_t)mb.size();
        d.modes_c = mc.data(); d.n_modes_c = (int32_t)mc.size();
        HostTensor A, B, C, Cref;
        A.init(dt, da, rng.below(5), rng);
        const bool two = kind == 2 || kind == 3;
        if (two) B.init(dt, db, rng.below(5), rng);
        const int lc = rng.below(4);
        Rng copy = rng;
        C.init(dt, dc, lc, rng);
        Cref.init(dt, dc, lc, copy);
        Cref.copy_data_from(C);
        std::vector<const int64_t*> shapes = {da.data()};
        std::vector<int32_t> ranks = {(int32_t)da.size()};
        if (two) { shapes.push_back(db.data()); ranks.push_back((int32_t)db.size()); }
        shapes.push_back(dc.data()); ranks.push_back((int32_t)dc.size());
        tfh_plan* plan = nullptr;
        const int32_t ps = tfh_plan_create(dt, &d, shapes.data(), ranks.data(), (int32_t)shapes.size(), &plan);
        CHECK(ps == TFH_OK);
        if (ps != TFH_OK) { tfh_error_info e; tfh_last_error(&e); std::printf("  plan kind %d: %s\n", kind, e.message); continue; }
        tfh_view in[2] = {A.view(), two ? B.view() : A.view()};
        tfh_view out = C.view();
        const int32_t es = tfh_execute(plan, alpha.ptr(dt), in, two ? 2 : 1, beta.ptr(dt), &out, nullptr);
        CHECK(es == TFH_OK);
        tfh_plan_destroy(plan);
        if (es != TFH_OK) { tfh_error_info e; tfh_last_error(&e); std::printf("  execute kind %d: %s\n", kind, e.message); continue; }
        tfo_view oa = A.oview(), ob = two ? B.oview() : A.oview(), oc = Cref.oview();
        int rc = 0;
        if (kind == 0) rc = tfo_permute(dt, alpha.ptr(dt), &oa, ma.data(), beta.ptr(dt), &oc, mc.data());
        else if (kind == 1) rc = tfo_reduce(dt, alpha.ptr(dt), &oa, ma.data(), beta.ptr(dt), &oc, mc.data(), d.reduce_op);
        else if (kind == 2) rc = tfo_contract(dt, alpha.ptr(dt), &oa, ma.data(), &ob, mb.data(), beta.ptr(dt), &oc, mc.data());
        else if (kind == 3) rc = tfo_elementwise_mul(dt, alpha.ptr(dt), &oa, &ob, beta.ptr(dt), &oc);
        else rc = tfo_trace(dt, alpha.ptr(dt), &oa, ma.data(), beta.ptr(dt), &oc, mc.data(), pair01, 1);
        CHECK(rc == 0);
        const double err = rel_err(C, Cref);
        CHECK(err < tol_of(dt));
        if (!(err < tol_of(dt))) std::printf("  kind %d dtype %d err %.3e\n", kind, dt, err);
    }
}

// ------------------------------------------------------------------------------------------------ routed launches kept in the plan
// A Contract plan keeps the routed launch of the first execute with each set of view strides (contract_cache.cpp): executes
// with strides it has seen run from the kept record, new strides route and are kept (eight sets, the oldest makes room),
// every result equals the oracle's, and threads that share one plan may execute it at the same time.
static void plan_keeps_routed_launches(Rng& rng) {
    const int dt = TFH_C128;
    const std::vector<uint32_t> ma = {0, 1, 2}, mb = {2, 3, 0}, mc = {0, 1, 3};   // batch 0, M 1, K 2, N 3
    const std::vector<int64_t> da = {3, 5, 4}, db = {4, 6, 3}, dc = {3, 5, 6};
    tfh_desc d;
    std::memset(&d, 0, sizeof d);
    d.op = TFH_OP_CONTRACT;
    d.modes_a = ma.data(); d.n_modes_a = 3;
    d.modes_b = mb.data(); d.n_modes_b = 3;
    d.modes_c = mc.data(); d.n_modes_c = 3;
    const int64_t* shapes[3] = {da.data(), db.data(), dc.data()};
    const int32_t ranks[3] = {3, 3, 3};
    tfh_plan* plan = nullptr;
    CHECK(tfh_plan_create(dt, &d, shapes, ranks, 3, &plan) == TFH_OK);
    if (!plan) return;
    const ScalarBytes alpha = scalar(dt, 0.75, -0.5), beta = scalar(dt, 0.25, 1.0);
    auto run = [&](int la, int lb, int lc, Rng& r) {
        HostTensor A, B, C, Cref;
        A.init(dt, da, la, r);
        B.init(dt, db, lb, r);
        Rng copy = r;
        C.init(dt, dc, lc, r);
        Cref.init(dt, dc, lc, copy);
        Cref.copy_data_from(C);
        tfh_view in[2] = {A.view(), B.view()};
        tfh_view out = C.view();
        CHECK(tfh_execute(plan, alpha.ptr(dt), in, 2, beta.ptr(dt), &out, nullptr) == TFH_OK);
        tfo_view oa = A.oview(), ob = B.oview(), oc = Cref.oview();
        CHECK(tfo_contract(dt, alpha.ptr(dt), &oa, ma.data(), &ob, mb.data(), beta.ptr(dt), &oc, mc.data()) == 0);
        CHECK(rel_err(C, Cref) < 1e-12);
    };
    int64_t hits = 0, misses = 0;
    int32_t entries = 0;
    const int64_t replays0 = tfh::host_backend_replays();
    // row-major everywhere, three times: one route, two replays (fresh buffers every time: only the strides are the key)
    for (int i = 0; i < 3; ++i) run(0, 0, 0, rng);
    CHECK(tfh_plan_cache_stats(plan, &hits, &misses, &entries) == TFH_OK && hits == 2 && misses == 1 && entries == 1);
    CHECK(tfh::host_backend_replays() - replays0 == 2);
    // column-major operands: new strides, a route of their own
    for (int i = 0; i < 2; ++i) run(1, 1, 0, rng);
    CHECK(tfh_plan_cache_stats(plan, &hits, &misses, &entries) == TFH_OK && hits == 3 && misses == 2 && entries == 2);
    // many random layouts: never more than eight routes kept, every result right, old routes make room
    for (int i = 0; i < 60; ++i) run(2 + rng.below(3), 2 + rng.below(3), rng.below(4), rng);
    CHECK(tfh_plan_cache_stats(plan, &hits, &misses, &entries) == TFH_OK && entries <= 8 && hits + misses == 65);
    // another alpha / beta class (beta == 0 overwrites) is a route of its own
    {
        HostTensor A, B, C;
        A.init(dt, da, 0, rng); B.init(dt, db, 0, rng); C.init(dt, dc, 0, rng);
        const ScalarBytes one = scalar(dt, 1, 0), zero = scalar(dt, 0, 0);
        tfh_view in[2] = {A.view(), B.view()};
        tfh_view out = C.view();
        int64_t m0 = 0, m1 = 0;
        tfh_plan_cache_stats(plan, nullptr, &m0, nullptr);
        CHECK(tfh_execute(plan, one.ptr(dt), in, 2, zero.ptr(dt), &out, nullptr) == TFH_OK);
        tfh_plan_cache_stats(plan, nullptr, &m1, nullptr);
        CHECK(m1 == m0 + 1);
    }
    // four threads on the one plan, each alternating between two layouts
    std::vector<std::thread> th;
    for (int t = 0; t < 4; ++t)
        th.emplace_back([&, t]() {
            Rng mine(1000 + t);
            for (int i = 0; i < 40; ++i) run((i + t) & 1, (i >> 1) & 1, 0, mine);
        });
    for (auto& x : th) x.join();
    CHECK(tfh_plan_cache_stats(plan, &hits, &misses, &entries) == TFH_OK && entries <= 8 && hits > 100);
    // no cache for other operations; null pointers are taken
    CHECK(tfh_plan_cache_stats(plan, nullptr, nullptr, nullptr) == TFH_OK && tfh_plan_cache_stats(nullptr, &hits, &misses, &entries) != TFH_OK);
    tfh_plan_destroy(plan);
}

// ------------------------------------------------------------------------------------------------ einsum executor vs the oracle
static void einsum_against_oracle(Rng& rng) {
    for (int iter = 0; iter < 300; ++iter) {
        const int dt = rng.below(4);
        const int n = 1 + rng.below(6);
        const int nlabels = 2 + rng.below(6);
        std::vector<int64_t> ext(nlabels);
        for (auto& e : ext) e = 1 + rng.below(4);
        std::vector<std::vector<uint32_t>> labs(n);
        std::vector<bool> used(nlabels, false);
        for (int i = 0; i < n; ++i) {
            for (int l = 0; l < nlabels; ++l)
                if (rng.below(5) < 2 && labs[i].size() < 4) { labs[i].push_back((uint32_t)l); used[l] = true; }
            for (int k = (int)labs[i].size() - 1; k > 0; --k) std::swap(labs[i][k], labs[i][rng.below(k + 1)]);
        }
        std::vector<uint32_t> out;
        for (int l = 0; l < nlabels; ++l) if (used[l] && rng.below(2)) out.push_back((uint32_t)l);
        for (int k = (int)out.size() - 1; k > 0; --k) std::swap(out[k], out[rng.below(k + 1)]);
        std::vector<uint32_t> flat;
        std::vector<int32_t> ranks(n);
        std::vector<HostTensor> ops(n);
        std::vector<std::vector<int64_t>> dims(n);
        std::vector<const int64_t*> ptrs(n);
        uint64_t donate = 0;
        for (int i = 0; i < n; ++i) {
            for (uint32_t l : labs[i]) { flat.push_back(l); dims[i].push_back(ext[l]); }
            if (dims[i].empty()) dims[i].reserve(1);
            ranks[i] = (int32_t)labs[i].size();
            ptrs[i] = dims[i].data();
            const bool give = rng.below(3) == 0;
            ops[i].init(dt, std::vector<int64_t>(dims[i].begin(), dims[i].begin() + ranks[i]), give ? rng.below(3) : rng.below(5), rng);
            if (give) donate |= 1ull << i;
        }
        std::vector<int64_t> od;
        for (uint32_t l : out) od.push_back(ext[l]);
        HostTensor C, Cref;
        const int lc = rng.below(4);
        Rng copy = rng;
        C.init(dt, od, lc, rng);
        Cref.init(dt, od, lc, copy);
        Cref.copy_data_from(C);
        const ScalarBytes alpha = scalar(dt, 0.5 + rng.uniform(), rng.uniform()), beta = rng.below(2) ? scalar(dt, rng.uniform(), rng.uniform()) : scalar(dt, 0, 0);
        // some complex operands are read through the conjugate-on-load flag; the reference gets a conjugated copy
        std::vector<HostTensor> conj_copies(n);
        std::vector<bool> flagged(n, false);
        for (int i = 0; i < n; ++i)
            if (is_cx(dt) && rng.below(4) == 0) { flagged[i] = true; conj_copies[i].conj_clone_of(ops[i]); }
        // the reference first: donated operands may be overwritten by the call under test
        std::vector<tfo_view> ov(n);
        for (int i = 0; i < n; ++i) ov[i] = flagged[i] ? conj_copies[i].oview() : ops[i].oview();
        tfo_view oc = Cref.oview();
        const int rc = tfo_einsum_naive(dt, n, ov.data(), flat.data(), ranks.data(), out.data(), (int)out.size(), alpha.ptr(dt), beta.ptr(dt), &oc);
        CHECK(rc == 0);
        tfh_subscripts* subs = nullptr;
        CHECK(tfh_subscripts_new(flat.data(), ranks.data(), n, out.data(), (int32_t)out.size(), &subs) == TFH_OK);
        if (!subs) continue;
        tfh_tree* tree = nullptr;
        const int32_t ts = (iter % 3 == 0) ? tfh_tree_optimize_cached(subs, ptrs.data(), ranks.data(), n, &tree)
                                           : tfh_tree_optimize(subs, ptrs.data(), ranks.data(), n, &tree);
        CHECK(ts == TFH_OK && tree);
        if (tree) {
            std::vector<tfh_view> views(n);
            for (int i = 0; i < n; ++i) { views[i] = ops[i].view(); if (flagged[i]) views[i].flags = TFH_VIEW_CONJ; }
            tfh_view outv = C.view();
            const int32_t es = tfh_einsum_execute(dt, tree, views.data(), n, alpha.ptr(dt), beta.ptr(dt), &outv, donate, nullptr);
            CHECK(es == TFH_OK);
            if (es == TFH_OK) {
                const double err = rel_err(C, Cref);
                CHECK(err < tol_of(dt) * 4);
                if (!(err < tol_of(dt) * 4)) std::printf("  einsum iter %d dtype %d n %d err %.3e\n", iter, dt, n, err);
            } else { tfh_error_info e; tfh_last_error(&e); std::printf("  einsum iter %d: %s\n", iter, e.message); }
            CHECK(tfh_tree_mac_count(tree) >= 0 && tfh_tree_peak_intermediate(tree) >= 0);
            tfh_tree_destroy(tree);
        }
        tfh_subscripts_destroy(subs);
        CHECK(tfh::host_backend_live_blocks() == 0);   // every intermediate was given back
    }
    // the pattern catalogue with repeated labels (tenferro-einsum/src/lib.rs:37-93) and an explicit order
    const char* patterns[] = {"ii->", "ii->i", "i->ii", "i->iii", "iij->j", "ij,ji->", "ij,(jk,kl)->il", "ab,bc,cd,de->ae", "a,a,a->a", "ab->"};
    for (const char* pat : patterns) {
        tfh_subscripts* subs = nullptr;
        CHECK(tfh_subscripts_parse(pat, &subs) == TFH_OK);
        if (!subs) continue;
        const int n = tfh_subscripts_n_inputs(subs);
        std::vector<uint32_t> flat, out(TFH_MAX_RANK);
        std::vector<int32_t> ranks(n);
        std::vector<HostTensor> ops(n);
        std::vector<std::vector<int64_t>> dims(n);
        std::vector<const int64_t*> ptrs(n);
        for (int i = 0; i < n; ++i) {
            uint32_t lab[TFH_MAX_RANK];
            ranks[i] = tfh_subscripts_labels(subs, i, lab, TFH_MAX_RANK);
            for (int k = 0; k < ranks[i]; ++k) { flat.push_back(lab[k]); dims[i].push_back(3); }
            if (dims[i].empty()) dims[i].reserve(1);
            ptrs[i] = dims[i].data();
            ops[i].init(TFH_C128, std::vector<int64_t>(dims[i].begin(), dims[i].begin() + ranks[i]), rng.below(4), rng);
        }
        const int no = tfh_subscripts_labels(subs, -1, out.data(), TFH_MAX_RANK);
        HostTensor C, Cref;
        Rng copy = rng;
        C.init(TFH_C128, std::vector<int64_t>(no, 3), 0, rng);
        Cref.init(TFH_C128, std::vector<int64_t>(no, 3), 0, copy);
        const ScalarBytes alpha = scalar(TFH_C128, 1.25, -0.5), beta = scalar(TFH_C128, 0, 0);
        std::vector<tfo_view> ov(n);
        for (int i = 0; i < n; ++i) ov[i] = ops[i].oview();
        tfo_view oc = Cref.oview();
        CHECK(tfo_einsum_naive(TFH_C128, n, ov.data(), flat.data(), ranks.data(), out.data(), no, alpha.ptr(TFH_C128), beta.ptr(TFH_C128), &oc) == 0);
        tfh_tree* tree = nullptr;
        CHECK(tfh_tree_optimize(subs, ptrs.data(), ranks.data(), n, &tree) == TFH_OK);
        if (tree) {
            std::vector<tfh_view> views(n);
            for (int i = 0; i < n; ++i) views[i] = ops[i].view();
            tfh_view outv = C.view();
            const int32_t es = tfh_einsum_execute(TFH_C128, tree, views.data(), n, alpha.ptr(TFH_C128), beta.ptr(TFH_C128), &outv, 0, nullptr);
            CHECK(es == TFH_OK);
            if (es == TFH_OK) CHECK(rel_err(C, Cref) < 1e-12);
            else { tfh_error_info e; tfh_last_error(&e); std::printf("  pattern %s: %s\n", pat, e.message); }
            tfh_tree_destroy(tree);
        }
        tfh_subscripts_destroy(subs);
    }
}

// ------------------------------------------------------------------------------------------------ trees
static void trees(Rng& rng) {
    tfh_subscripts* subs = nullptr;
    CHECK(tfh_subscripts_parse("ab,bc,cd,de->ae", &subs) == TFH_OK);
    const int64_t d[2] = {3, 3};
    const int64_t* shapes[4] = {d, d, d, d};
    const int32_t ranks[4] = {2, 2, 2, 2};
    // from_pairs: a valid order, then orders that reuse an operand, name one that does not exist yet, or stop early
    const int32_t ok[6] = {0, 1, 2, 3, 4, 5};
    tfh_tree* t = nullptr;
    CHECK(tfh_tree_from_pairs(subs, shapes, ranks, 4, ok, 3, &t) == TFH_OK && t);
    if (t) {
        CHECK(tfh_tree_n_inputs(t) == 4 && tfh_tree_n_steps(t) == 3 && tfh_tree_output_rank(t) == 2);
        int32_t l = -1, r = -1;
        CHECK(tfh_tree_step(t, 2, &l, &r) == TFH_OK && l == 4 && r == 5);
        CHECK(tfh_tree_step(t, 3, &l, &r) != TFH_OK && tfh_tree_step(t, -1, &l, &r) != TFH_OK);
        tfh_tree_destroy(t);
    }
    const int32_t bads[][6] = {{0, 1, 0, 2, 4, 5}, {0, 1, 2, 9, 4, 5}, {0, 1, 2, 3, 4, 4}, {0, 5, 2, 3, 4, 5}, {-1, 1, 2, 3, 4, 5}};
    for (auto& b : bads) {
        t = nullptr;
        CHECK(tfh_tree_from_pairs(subs, shapes, ranks, 4, b, 3, &t) != TFH_OK && t == nullptr);
    }
    t = nullptr;
    CHECK(tfh_tree_from_pairs(subs, shapes, ranks, 4, ok, 2, &t) != TFH_OK && t == nullptr);
    CHECK(tfh_tree_optimize(subs, shapes, ranks, 3, &t) != TFH_OK);   // wrong operand count
    const int32_t wrong_ranks[4] = {2, 3, 2, 2};
    CHECK(tfh_tree_optimize(subs, shapes, wrong_ranks, 4, &t) != TFH_OK);
    tfh_subscripts_destroy(subs);

    // the shared tree cache from four threads, with more distinct networks than it keeps (512): entries are evicted
    // while other threads still hold and use them
    tfh_tree_cache_clear();
    auto worker = [](int id) {
        Rng r(1000 + id);
        tfh_subscripts* s = nullptr;
        if (tfh_subscripts_parse("ab,bc,cd->ad", &s) != TFH_OK) return;
        std::vector<tfh_tree*> held;
        for (int i = 0; i < 400; ++i) {
            const int64_t a[2] = {1 + r.below(30), 1 + r.below(30)}, b[2] = {a[1], 1 + r.below(30)}, c[2] = {b[1], 1 + r.below(4)};
            const int64_t* sh[3] = {a, b, c};
            const int32_t rk[3] = {2, 2, 2};
            tfh_tree* tr = nullptr;
            if (tfh_tree_optimize_cached(s, sh, rk, 3, &tr) == TFH_OK && tr) held.push_back(tr);
            if (held.size() > 50) {
                (void)tfh_tree_mac_count(held.front());
                tfh_tree_destroy(held.front());
                held.erase(held.begin());
            }
        }
        for (tfh_tree* tr : held) { (void)tfh_tree_n_steps(tr); tfh_tree_destroy(tr); }
        tfh_subscripts_destroy(s);
    };
    std::vector<std::thread> threads;
    for (int i = 0; i < 4; ++i) threads.emplace_back(worker, i);
    for (auto& th : threads) th.join();
    int64_t hits = 0, misses = 0, entries = 0;
    CHECK(tfh_tree_cache_stats(&hits, &misses, &entries) == TFH_OK && entries <= 512 && hits + misses == 1600);
    CHECK(tfh_tree_cache_clear() == TFH_OK);
    (void)rng;
}

// ------------------------------------------------------------------------------------------------ the oracle by itself
static void oracle_blocked_against_brute_force(Rng& rng) {
    // sizes past one cache block in every direction, odd remainders, all four dtypes, both with and without beta
    struct Case { int64_t m, n, k, b; };
    const Case cases[] = {{150, 131, 140, 1}, {37, 260, 19, 2}, {300, 5, 77, 1}, {1, 1, 1000, 3}, {64, 64, 64, 1}};
    for (int dt = 0; dt < 4; ++dt)
        for (const Case& c : cases) {
            HostTensor A, B, C, Cref;
            A.init(dt, {c.b, c.m, c.k}, rng.below(4), rng);
            B.init(dt, {c.k, c.b, c.n}, rng.below(4), rng);
            const int lc = rng.below(2);
            Rng copy = rng;
            C.init(dt, {c.m, c.n, c.b}, lc, rng);
            Cref.init(dt, {c.m, c.n, c.b}, lc, copy);
            Cref.copy_data_from(C);
            const uint32_t ma[3] = {0, 1, 3}, mb[3] = {3, 0, 2}, mc[3] = {1, 2, 0};
            const ScalarBytes alpha = scalar(dt, 0.75, 0.25), beta = scalar(dt, -0.5, 0.125);
            tfo_view oa = A.oview(), ob = B.oview(), oc = C.oview(), orf = Cref.oview();
            CHECK(tfo_contract(dt, alpha.ptr(dt), &oa, ma, &ob, mb, beta.ptr(dt), &oc, mc) == 0);
            CHECK(tfo_contract_naive(dt, alpha.ptr(dt), &oa, ma, &ob, mb, beta.ptr(dt), &orf, mc) == 0);
            const double err = rel_err(C, Cref);
            CHECK(err < tol_of(dt));
            if (!(err < tol_of(dt))) std::printf("  oracle dtype %d m %lld n %lld k %lld err %.3e\n", dt, (long long)c.m, (long long)c.n, (long long)c.k, err);
        }
    // the other oracle routines on ragged shapes and strided views (their loops, under the sanitizers)
    for (int iter = 0; iter < 60; ++iter) {
        const int dt = rng.below(4);
        HostTensor A, P, R, T, At, Ad;
        const int64_t a = 1 + rng.below(7), b = 1 + rng.below(7), c = 1 + rng.below(7);
        A.init(dt, {a, b, c}, rng.below(5), rng);
        P.init(dt, {c, a, b}, rng.below(4), rng);
        R.init(dt, {b}, rng.below(2), rng);
        const uint32_t m3[3] = {0, 1, 2}, mp[3] = {2, 0, 1}, mr[1] = {1};
        const ScalarBytes one = scalar(dt, 1, 0), zero = scalar(dt, 0, 0);
        tfo_view oa = A.oview(), op = P.oview(), orr = R.oview();
        CHECK(tfo_permute(dt, one.ptr(dt), &oa, m3, zero.ptr(dt), &op, mp) == 0);
        CHECK(tfo_reduce(dt, one.ptr(dt), &oa, m3, zero.ptr(dt), &orr, mr, TFO_SUM) == 0);
        HostTensor S, D3;
        S.init(dt, {a, a, c}, rng.below(5), rng);
        T.init(dt, {c}, 0, rng);
        At.init(dt, {a, a, c}, rng.below(4), rng);
        Ad.init(dt, {a, c}, rng.below(4), rng);
        D3.init(dt, {a, a, c}, rng.below(4), rng);
        const uint32_t mt[1] = {2}, pair[2] = {0, 1}, md[2] = {0, 2};
        tfo_view os = S.oview(), ot = T.oview(), oat = At.oview(), oad = Ad.oview(), od3 = D3.oview();
        CHECK(tfo_trace(dt, one.ptr(dt), &os, m3, zero.ptr(dt), &ot, mt, pair, 1) == 0);
        CHECK(tfo_anti_trace(dt, one.ptr(dt), &ot, mt, zero.ptr(dt), &oat, m3, pair, 1) == 0);
        CHECK(tfo_anti_diag(dt, one.ptr(dt), &oad, md, zero.ptr(dt), &od3, m3, pair, 1) == 0);
        CHECK(tfo_conj(dt, &oa, &oa) == 0);
    }
}

int main() {
    Rng rng(20240607);
    tfo_set_num_threads(4);
    error_records();
    parser_cases(rng);
    plan_validation(rng);
    trees(rng);
    prims_against_oracle(rng);
    plan_keeps_routed_launches(rng);
    einsum_against_oracle(rng);
    oracle_blocked_against_brute_force(rng);
    tfh_tree_cache_clear();
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed ? 1 : 0;
}
