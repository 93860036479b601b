// contract_cache.cpp -- kernel selection kept with the plan (tenferro-prims/src/lib.rs:8 "Build a plan via
// TensorPrims::plan (pre-computes kernel selection)", :284 "The plan pre-computes kernel selection and workspace sizes").
//
// What a contraction's route depends on, besides the extents, only shows when the views arrive: their strides.  So the
// plan keeps, per set of strides it has been executed with, the routed launch the first such call produced (the
// launcher's ContractRecord); a later execute with the same strides looks it up, patches addresses and scalars into it
// and enqueues -- no axis classification, no fusion, no tile or split choice, no heap allocation.  The steps of an einsum
// tree keep the same cache.  Pure host code.
#include <cstring>
#include <mutex>

#include "internal.hpp"

namespace tfh {
namespace {
struct Key {
    int32_t n = 0;
    int64_t v[3 * TFH_MAX_RANK + 2];
    bool operator==(const Key& o) const { return n == o.n && std::memcmp(v, o.v, sizeof(int64_t) * (size_t)n) == 0; }
};
}  // namespace

struct ContractCache {
    static constexpr int WAYS = 8;   // stride sets per plan; the oldest entry makes room
    struct Entry {
        Key key;
        std::shared_ptr<ContractRecord> rec;
    };
    mutable std::mutex mu;
    Entry e[WAYS];
    int used = 0, next = 0;
    int64_t hits = 0, misses = 0;
};

ContractCache* contract_cache_create() { return new (std::nothrow) ContractCache(); }
void contract_cache_destroy(ContractCache* c) { delete c; }
void contract_cache_stats(const ContractCache* c, int64_t* hits, int64_t* misses, int32_t* entries) {
    int64_t h = 0, m = 0;
    int32_t n = 0;
    if (c) {
        std::lock_guard<std::mutex> lk(c->mu);
        h = c->hits;
        m = c->misses;
        n = c->used;
    }
    if (hits) *hits = h;
    if (misses) *misses = m;
    if (entries) *entries = n;
}

std::string contract_cache_routes(const ContractCache* c) {
    std::string r;
    if (!c) return r;
    std::lock_guard<std::mutex> lk(c->mu);
    for (int i = 0; i < c->used; ++i) {
        if (!c->e[i].rec) continue;
        if (!r.empty()) r += "; ";
        r += c->e[i].rec->label;
    }
    return r;
}

int32_t execute_contract(ContractCache* cache, int dtype, const std::vector<uint32_t>& ma, const int64_t* dims_a, const int64_t* str_a,
                         const void* a, const std::vector<uint32_t>& mb, const int64_t* dims_b, const int64_t* str_b, const void* b,
                         const std::vector<uint32_t>& mc, const int64_t* dims_c, const int64_t* str_c, void* c, Scalar alpha,
                         Scalar beta, void* stream, int conj) {
    Key key;
    std::shared_ptr<ContractRecord> rec;
    if (cache) {
        for (size_t d = 0; d < ma.size(); ++d) key.v[key.n++] = str_a[d];
        for (size_t d = 0; d < mb.size(); ++d) key.v[key.n++] = str_b[d];
        for (size_t d = 0; d < mc.size(); ++d) key.v[key.n++] = str_c[d];
        key.v[key.n++] = (int64_t)(((uintptr_t)a & 15) | (((uintptr_t)b & 15) << 4) | (((uintptr_t)c & 15) << 8) |
                                   ((uint64_t)(conj & 3) << 12) | ((uint64_t)(beta.is_zero() ? 1 : 0) << 14) |
                                   ((uint64_t)((alpha.re == 1.0 && alpha.im == 0.0) ? 1 : 0) << 15) | ((uint64_t)(dtype & 15) << 16));
        key.v[key.n++] = (int64_t)(uintptr_t)stream;
        {
            std::lock_guard<std::mutex> lk(cache->mu);
            for (int i = 0; i < cache->used; ++i)
                if (cache->e[i].key == key) {
                    rec = cache->e[i].rec;
                    break;
                }
            if (rec) ++cache->hits;
            else ++cache->misses;
        }
        if (rec) {
            int32_t status = TFH_OK;
            if (replay_contract(*rec, dtype, a, b, c, alpha, beta, stream, status)) return status;
            // the record went stale (its tables were released): forget it and route the call again
            std::lock_guard<std::mutex> lk(cache->mu);
            for (int i = 0; i < cache->used; ++i)
                if (cache->e[i].rec == rec) {
                    cache->e[i] = cache->e[cache->used - 1];
                    cache->e[cache->used - 1].rec.reset();
                    --cache->used;
                    break;
                }
            rec.reset();
        }
    }
    ContractAxes ax;
    if (int32_t e = classify_contract(ma, dims_a, str_a, mb, dims_b, str_b, mc, dims_c, str_c, ax)) return e;
    std::shared_ptr<ContractRecord> made;
    const int32_t e = launch_contract(dtype, a, b, c, ax, alpha, beta, stream, conj, cache ? &made : nullptr);
    if (!e && made) {
        std::lock_guard<std::mutex> lk(cache->mu);
        bool present = false;
        for (int i = 0; i < cache->used; ++i) present = present || cache->e[i].key == key;
        if (!present) {   // (another thread may have routed the same strides meanwhile)
            const int at = cache->used < ContractCache::WAYS ? cache->used++ : (cache->next++ % ContractCache::WAYS);
            cache->e[at].key = key;
            cache->e[at].rec = std::move(made);
        }
    }
    return e;
}

}  // namespace tfh
