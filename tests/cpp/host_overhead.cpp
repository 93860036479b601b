// host_overhead.cpp -- microseconds of host time per tfh_execute enqueue, measured from C (no interpreter in the loop):
// the first execute of a plan (routing, tables, workspace) against repeated ones, which find the routed launch in the
// plan (tenferro-prims/src/lib.rs:8, :284: "the plan pre-computes kernel selection").  Host compiler only; links the C ABI.
//
//   ./host_overhead        (run by `python3 bench.py --host-overhead`)
//
// Bursts of 200 calls on an idle stream, so that the launch queue never fills and the host is never held back by the
// device; the best of five bursts.  "with drain" adds the wait for the device: when it is the larger figure by far the
// stream, not the host, sets the pace.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../../include/tenferro_hip.h"

static double now() { return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

static tfh_view dense(void* base, const std::vector<int64_t>& dims) {
    tfh_view v;
    std::memset(&v, 0, sizeof v);
    v.base = base;
    v.rank = (int32_t)dims.size();
    int64_t run = 1;
    for (int d = (int)dims.size() - 1; d >= 0; --d) {
        v.dims[d] = dims[d];
        v.strides[d] = run;
        run *= dims[d];
    }
    return v;
}

struct Case {
    const char* name;
    int dtype;
    std::vector<uint32_t> ma, mb, mc;
    std::vector<int64_t> da, db, dc;
};

int main() {
    tfh_stream st = nullptr;
    if (tfh_stream_create(&st)) { std::printf("no device\n"); return 1; }
    const Case cases[] = {
        {"Contract ij,jk->ik f64 64^3 (one launch)", TFH_F64, {0, 1}, {1, 2}, {0, 2}, {64, 64}, {64, 64}, {64, 64}},
        {"Contract ij,jk->ik f64 128^3 (split-K + fold: two launches)", TFH_F64, {0, 1}, {1, 2}, {0, 2}, {128, 128}, {128, 128}, {128, 128}},
        {"Contract ij,jk->ik f64 1024^3 (one launch)", TFH_F64, {0, 1}, {1, 2}, {0, 2}, {1024, 1024}, {1024, 1024}, {1024, 1024}},
        {"configuration 1: ajbk,kcj->abc f32 (pack of B, tables, split-K)", TFH_F32, {0, 1, 2, 3}, {3, 4, 1}, {0, 2, 4}, {64, 128, 64, 96}, {96, 256, 128}, {64, 64, 256}},
    };
    for (const Case& c : cases) {
        tfh_desc d;
        std::memset(&d, 0, sizeof d);
        d.op = TFH_OP_CONTRACT;
        d.modes_a = c.ma.data(); d.n_modes_a = (int32_t)c.ma.size();
        d.modes_b = c.mb.data(); d.n_modes_b = (int32_t)c.mb.size();
        d.modes_c = c.mc.data(); d.n_modes_c = (int32_t)c.mc.size();
        const int64_t* shapes[3] = {c.da.data(), c.db.data(), c.dc.data()};
        const int32_t ranks[3] = {(int32_t)c.da.size(), (int32_t)c.db.size(), (int32_t)c.dc.size()};
        tfh_plan* plan = nullptr;
        if (tfh_plan_create(c.dtype, &d, shapes, ranks, 3, &plan)) { std::printf("plan failed\n"); return 1; }
        auto count = [](const std::vector<int64_t>& v) { size_t n = 1; for (int64_t x : v) n *= (size_t)x; return n; };
        const size_t eb = tfh_dtype_size(c.dtype);
        void *A = nullptr, *B = nullptr, *C = nullptr;
        if (tfh_malloc(count(c.da) * eb, &A) || tfh_malloc(count(c.db) * eb, &B) || tfh_malloc(count(c.dc) * eb, &C)) { std::printf("out of memory\n"); return 1; }
        std::vector<char> zeros(std::max(count(c.da), count(c.db)) * eb, 0);
        tfh_memcpy_h2d(A, zeros.data(), count(c.da) * eb, st);
        tfh_memcpy_h2d(B, zeros.data(), count(c.db) * eb, st);
        tfh_stream_synchronize(st);
        tfh_view in[2] = {dense(A, c.da), dense(B, c.db)};
        tfh_view out = dense(C, c.dc);
        const double one64 = 1.0, zero64 = 0.0;
        const float one32 = 1.0f, zero32 = 0.0f;
        const void* al = c.dtype == TFH_F32 ? (const void*)&one32 : (const void*)&one64;
        const void* be = c.dtype == TFH_F32 ? (const void*)&zero32 : (const void*)&zero64;
        double t0 = now();
        if (tfh_execute(plan, al, in, 2, be, &out, st)) { std::printf("execute failed\n"); return 1; }
        const double first = (now() - t0) * 1e6;
        tfh_stream_synchronize(st);
        for (int i = 0; i < 20; ++i) tfh_execute(plan, al, in, 2, be, &out, st);
        tfh_stream_synchronize(st);
        const int N = 200;
        double best = 1e30, best_drain = 0;
        for (int rep = 0; rep < 5; ++rep) {
            t0 = now();
            for (int i = 0; i < N; ++i) tfh_execute(plan, al, in, 2, be, &out, st);
            const double t1 = now();
            tfh_stream_synchronize(st);
            const double t2 = now();
            if ((t1 - t0) < best) { best = t1 - t0; best_drain = t2 - t0; }
        }
        int64_t hits = 0, misses = 0;
        int32_t entries = 0;
        tfh_plan_cache_stats(plan, &hits, &misses, &entries);
        std::printf("%-66s first call %8.1f us   repeated enqueue %5.2f us   with drain %7.2f us   routes found/made/kept %lld/%lld/%d   %s\n", c.name, first,
                    best * 1e6 / N, best_drain * 1e6 / N, (long long)hits, (long long)misses, (int)entries, tfh_last_kernel());
        tfh_plan_destroy(plan);
        tfh_free(A); tfh_free(B); tfh_free(C);
    }
    tfh_stream_destroy(st);
    return 0;
}
