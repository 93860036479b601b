// runtime.cpp -- device, memory, stream and event entry points of the C ABI plus the per-stream
// scratch memory the kernels use.  Mirrors the device model of tenferro-device/src/lib.rs:30-105 and
// the GPU-async vocabulary of tenferro-tensor/src/lib.rs:301-309, 660-713.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>
#include <atomic>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "internal.hpp"

namespace tfh {

int32_t hip_check(int err, const char* what) {
    if (err == hipSuccess) return TFH_OK;
    return set_error(TFH_ERR_DEVICE, "%s: %s", what, hipGetErrorString((hipError_t)err));
}

namespace {
// A buffer that was handed out while its stream was being captured into a graph is part of that graph: replays read
// and write it long after the call that took it has returned.  Such buffers are "pinned": nothing here frees them
// before the process ends (a workspace that has to grow is retired instead of freed, tfh_release_workspaces and the
// out-of-memory path pass them over).  Pinned blocks still serve later calls on their stream, which stream order keeps
// apart from a replay launched into the same stream.
struct StreamScratch {
    void* ws = nullptr;
    size_t ws_bytes = 0;
    bool ws_pinned = false;
    std::vector<void*> retired;                 // pinned workspaces that were outgrown
    std::multimap<size_t, void*> free_blocks;   // cached intermediates by size
    std::map<void*, size_t> live;
    std::set<void*> pinned_blocks;              // intermediates handed out during a capture
    // offset tables of contractions already run on this stream, by the dims and strides they were built from
    struct Tables { void* dev; size_t bytes; bool filled; bool pinned; };
    std::map<std::string, Tables> tables;
    size_t table_bytes = 0;
    // two pinned host buffers for transfers from and to pageable host memory (allocated on first use)
    // One staged transfer at a time uses them: bounce_mu is held from a transfer's first chunk to its last, so two host
    // threads that copy pageable memory on one stream take turns instead of filling each other's staging buffers.
    std::mutex bounce_mu;
    void* bounce[2] = {nullptr, nullptr};
    hipEvent_t bounce_ev[2] = {nullptr, nullptr};
    bool bounce_busy[2] = {false, false};   // a copy recorded in bounce_ev may still be using the buffer
};
// Buffers that a captured graph may still use when their stream is destroyed: kept until the process ends.
std::vector<void*> g_orphans;
constexpr size_t BOUNCE_BYTES = (size_t)16 << 20;
bool capturing(void* stream) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return cs != hipStreamCaptureStatusNone;
}
constexpr size_t TABLE_CACHE_BYTES = (size_t)64 << 20;   // per stream; beyond it tables go to the workspace again
constexpr size_t TABLE_CACHE_ENTRIES = 256;
std::mutex g_mu;
std::map<std::pair<int, void*>, StreamScratch> g_scratch;   // (device, stream)
std::atomic<uint64_t> g_table_epoch{0};   // see table_epoch()

// While a call made through tfh_execute_static is running on this thread, every piece of device scratch it asks for
// (workspace, packed operands, offset tables) is carved out of a fixed region handed in by arena_begin(); nothing is
// allocated, cached or freed.
struct Arena {
    char* base = nullptr;
    size_t cap = 0, used = 0;
    bool active = false;
};
thread_local Arena t_arena;
int32_t arena_alloc(size_t bytes, void** out, const char* what) {
    const size_t at = (t_arena.used + 255) & ~(size_t)255;
    if (bytes > t_arena.cap || at > t_arena.cap - bytes)
        return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: the call needs %zu bytes of scratch memory beyond the %zu already taken; the static scratch holds %zu",
                         what, bytes, at, t_arena.cap);
    *out = t_arena.base + at;
    t_arena.used = at + bytes;
    return TFH_OK;
}

StreamScratch* scratch_for(void* stream, int32_t* err) {
    int dev = 0;
    *err = hip_check(hipGetDevice(&dev), "hipGetDevice");
    if (*err) return nullptr;
    return &g_scratch[{dev, stream}];
}

// hipMalloc that, when the device is out of memory, gives back the blocks cached for reuse on every stream of the
// current device (after the work that may still read them has finished) and tries once more.  `stream`: the stream
// the caller enqueues on, checked for an ongoing graph capture (which forbids the synchronisation); g_mu is held.
int32_t malloc_or_release(void** p, size_t bytes, void* stream, const char* what) {
    if (hipMalloc(p, bytes) == hipSuccess) return TFH_OK;
    (void)hipGetLastError();
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return set_error(TFH_ERR_DEVICE, "%s: out of memory for %zu bytes while the stream is being captured", what, bytes);
    }
    if (int32_t e = hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize")) return e;
    int dev = 0;
    (void)hipGetDevice(&dev);
    for (auto& kv : g_scratch) {
        if (kv.first.first != dev) continue;
        auto& fb = kv.second.free_blocks;
        for (auto it = fb.begin(); it != fb.end();) {
            if (kv.second.pinned_blocks.count(it->second)) {
                ++it;
                continue;
            }
            (void)hipFree(it->second);
            it = fb.erase(it);
        }
    }
    return hip_check(hipMalloc(p, bytes), what);
}
}  // namespace

bool stream_is_capturing(void* stream) { return capturing(stream); }

void arena_begin(void* base, size_t bytes) { t_arena = Arena{(char*)base, bytes, 0, true}; }
void arena_end() { t_arena = Arena{}; }

int32_t workspace(void* stream, size_t bytes, void** out) {
    if (t_arena.active) return arena_alloc(bytes, out, "workspace");
    std::lock_guard<std::mutex> lk(g_mu);
    int32_t err;
    StreamScratch* s = scratch_for(stream, &err);
    if (!s) return err;
    const bool cap = capturing(stream);
    if (bytes > s->ws_bytes) {
        if (s->ws) {
            if (s->ws_pinned || cap) {
                // a captured graph holds the old buffer (or is being recorded right now, when nothing may wait): keep it
                s->retired.push_back(s->ws);
            } else {
                // kernels already enqueued may still read the old buffer
                if (int32_t e = hip_check(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize")) return e;
                (void)hipFree(s->ws);
            }
            s->ws = nullptr;
            s->ws_bytes = 0;
            s->ws_pinned = false;
        }
        size_t want = std::max<size_t>(bytes + bytes / 4, (size_t)1 << 20);
        if (int32_t e = malloc_or_release(&s->ws, want, stream, "hipMalloc(workspace)")) return e;
        s->ws_bytes = want;
    }
    if (cap) s->ws_pinned = true;
    *out = s->ws;
    return TFH_OK;
}

int32_t table_cache_get(void* stream, const std::string& key, size_t bytes, void** tables, bool* fresh) {
    *tables = nullptr;
    *fresh = false;
    if (t_arena.active) return TFH_OK;   // no cache in a call that must not allocate: the tables go to its workspace
    std::lock_guard<std::mutex> lk(g_mu);
    int32_t err;
    StreamScratch* s = scratch_for(stream, &err);
    if (!s) return err;
    auto it = s->tables.find(key);
    if (it != s->tables.end()) {
        if (it->second.filled && it->second.bytes == bytes) {
            *tables = it->second.dev;
            if (capturing(stream)) it->second.pinned = true;
        }
        return TFH_OK;
    }
    if (s->tables.size() >= TABLE_CACHE_ENTRIES || s->table_bytes + bytes > TABLE_CACHE_BYTES) return TFH_OK;
    // no new cache entry while the stream is being captured into a graph: the call then builds its tables in the workspace
    if (capturing(stream)) return TFH_OK;
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();   // out of memory for the cache is not an error of the call
        return TFH_OK;
    }
    s->tables[key] = StreamScratch::Tables{p, bytes, false, false};
    s->table_bytes += bytes;
    *tables = p;
    *fresh = true;
    return TFH_OK;
}

uint64_t table_epoch() { return g_table_epoch.load(std::memory_order_acquire); }

void table_cache_commit(void* stream, const std::string& key) {
    std::lock_guard<std::mutex> lk(g_mu);
    int32_t err;
    StreamScratch* s = scratch_for(stream, &err);
    if (!s) return;
    auto it = s->tables.find(key);
    if (it != s->tables.end()) it->second.filled = true;
}

int32_t pool_alloc(void* stream, size_t bytes, void** out) {
    if (t_arena.active) return arena_alloc(bytes, out, "packed operand");
    std::lock_guard<std::mutex> lk(g_mu);
    int32_t err;
    StreamScratch* s = scratch_for(stream, &err);
    if (!s) return err;
    bytes = std::max<size_t>((bytes + 255) & ~(size_t)255, 256);
    const bool cap = capturing(stream);
    auto it = s->free_blocks.lower_bound(bytes);
    if (it != s->free_blocks.end() && it->first <= bytes + bytes / 4) {
        *out = it->second;
        s->live[*out] = it->first;
        s->free_blocks.erase(it);
        if (cap) s->pinned_blocks.insert(*out);
        return TFH_OK;
    }
    void* p = nullptr;
    if (int32_t e = malloc_or_release(&p, bytes, stream, "hipMalloc(intermediate)")) return e;
    s->live[p] = bytes;
    if (cap) s->pinned_blocks.insert(p);
    *out = p;
    return TFH_OK;
}

void pool_free(void* stream, void* ptr) {
    if (!ptr || t_arena.active) return;   // arena blocks live until the call ends
    std::lock_guard<std::mutex> lk(g_mu);
    int32_t err;
    StreamScratch* s = scratch_for(stream, &err);
    if (!s) return;
    auto it = s->live.find(ptr);
    if (it == s->live.end()) return;
    // stream-ordered reuse: the next user of this block is enqueued on the same stream
    s->free_blocks.emplace(it->second, ptr);
    s->live.erase(it);
}

namespace {
// Is this host pointer page-locked memory the device can read and write directly?
bool is_pinned_host(const void* p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();   // ordinary (pageable) memory is unknown to the runtime
        return false;
    }
    return attr.type == hipMemoryTypeHost;
}

// The stream's scratch entry (entries of the map stay where they are until their stream is destroyed).
int32_t bounce_scratch(void* stream, StreamScratch** out) {
    std::lock_guard<std::mutex> lk(g_mu);
    int32_t err;
    StreamScratch* s = scratch_for(stream, &err);
    if (!s) return err;
    *out = s;
    return TFH_OK;
}
// The two staging buffers, allocated on first use; bounce_mu is held.
int32_t bounce_buffers(StreamScratch* s) {
    for (int i = 0; i < 2; ++i) {
        if (!s->bounce[i]) {
            if (int32_t e = hip_check(hipHostMalloc(&s->bounce[i], BOUNCE_BYTES, hipHostMallocDefault), "hipHostMalloc(staging buffer)")) return e;
            if (int32_t e = hip_check(hipEventCreateWithFlags(&s->bounce_ev[i], hipEventDisableTiming), "hipEventCreate")) return e;
            s->bounce_busy[i] = false;
        }
    }
    return TFH_OK;
}
// Frees the staging buffers of a scratch entry; no copy may be using them (the caller has synchronised).
void free_bounce(StreamScratch& sc) {
    std::lock_guard<std::mutex> lk(sc.bounce_mu);
    for (int i = 0; i < 2; ++i) {
        if (sc.bounce[i]) (void)hipHostFree(sc.bounce[i]);
        if (sc.bounce_ev[i]) (void)hipEventDestroy(sc.bounce_ev[i]);
        sc.bounce[i] = nullptr;
        sc.bounce_ev[i] = nullptr;
        sc.bounce_busy[i] = false;
    }
}

// Pageable host memory cannot be the source or target of an asynchronous copy: the transfer goes through two pinned
// staging buffers in chunks, the host filling (or emptying) one while the copy engine works on the other, so that the
// transfer proceeds at the engine's rate and runs beside kernels of other streams.  The call returns when the host side
// is done: for host-to-device, when the last chunk has been handed to the stream; for device-to-host, when the data is in
// `dst`.  Pinned memory (tfh_host_malloc) is copied directly and fully asynchronously.
int32_t wait_bounce(StreamScratch* s, int b) {
    if (!s->bounce_busy[b]) return TFH_OK;
    s->bounce_busy[b] = false;
    return hip_check(hipEventSynchronize(s->bounce_ev[b]), "hipEventSynchronize");
}
int32_t staged_h2d(void* dst, const void* src, size_t bytes, void* stream) {
    StreamScratch* s = nullptr;
    if (int32_t e = bounce_scratch(stream, &s)) return e;
    std::lock_guard<std::mutex> turn(s->bounce_mu);
    if (int32_t e = bounce_buffers(s)) return e;
    size_t done = 0;
    for (int i = 0; done < bytes; ++i) {
        const int b = i & 1;
        const size_t n = std::min(BOUNCE_BYTES, bytes - done);
        if (int32_t e = wait_bounce(s, b)) return e;   // the copy that last used this buffer (of this or an earlier call) has finished
        std::memcpy(s->bounce[b], (const char*)src + done, n);
        if (int32_t e = hip_check(hipMemcpyAsync((char*)dst + done, s->bounce[b], n, hipMemcpyHostToDevice, (hipStream_t)stream), "hipMemcpyAsync(h2d)")) return e;
        if (int32_t e = hip_check(hipEventRecord(s->bounce_ev[b], (hipStream_t)stream), "hipEventRecord")) return e;
        s->bounce_busy[b] = true;
        done += n;
    }
    return TFH_OK;
}
int32_t staged_d2h(void* dst, const void* src, size_t bytes, void* stream) {
    StreamScratch* s = nullptr;
    if (int32_t e = bounce_scratch(stream, &s)) return e;
    std::lock_guard<std::mutex> turn(s->bounce_mu);
    if (int32_t e = bounce_buffers(s)) return e;
    const size_t nchunks = (bytes + BOUNCE_BYTES - 1) / BOUNCE_BYTES;
    auto issue = [&](size_t c) {
        const int b = (int)(c & 1);
        const size_t at = c * BOUNCE_BYTES, n = std::min(BOUNCE_BYTES, bytes - at);
        if (int32_t e = wait_bounce(s, b)) return e;   // an earlier host-to-device copy may still be reading it
        if (int32_t e = hip_check(hipMemcpyAsync(s->bounce[b], (const char*)src + at, n, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync(d2h)")) return e;
        return hip_check(hipEventRecord(s->bounce_ev[b], (hipStream_t)stream), "hipEventRecord");
    };
    if (nchunks > 0)
        if (int32_t e = issue(0)) return e;
    for (size_t c = 0; c < nchunks; ++c) {
        if (c + 1 < nchunks)
            if (int32_t e = issue(c + 1)) return e;   // the engine fills the other buffer while the host empties this one
        const int b = (int)(c & 1);
        if (int32_t e = hip_check(hipEventSynchronize(s->bounce_ev[b]), "hipEventSynchronize")) return e;
        const size_t at = c * BOUNCE_BYTES, n = std::min(BOUNCE_BYTES, bytes - at);
        std::memcpy((char*)dst + at, s->bounce[b], n);
    }
    return TFH_OK;
}
}  // namespace

namespace {
struct ProfRec {
    int kind;
    hipEvent_t a, b;
    const char* name = "";   // label of the kernel that took the events (static storage)
};
std::mutex g_prof_mu;
bool g_prof_on = false;
std::vector<ProfRec> g_prof;
std::vector<hipEvent_t> g_prof_pool;
hipEvent_t prof_event() {
    if (!g_prof_pool.empty()) {
        hipEvent_t e = g_prof_pool.back();
        g_prof_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    (void)hipEventCreate(&e);
    return e;
}
}  // namespace

namespace {
thread_local ProfEvents t_pending;
thread_local const char* t_last_kernel = "";
}
void note_kernel(const char* name) { t_last_kernel = name; }
const char* last_kernel() { return t_last_kernel; }
int prof_begin(int kind, void* stream) {
    (void)stream;
    if (!g_prof_on) return -1;
    std::lock_guard<std::mutex> lk(g_prof_mu);
    ProfRec r{kind, prof_event(), prof_event()};
    if (!r.a || !r.b) return -1;
    t_pending.start = r.a;
    t_pending.stop = r.b;
    g_prof.push_back(r);
    return (int)g_prof.size() - 1;
}
ProfEvents prof_take(const char* name) {
    ProfEvents e = t_pending;
    t_pending = ProfEvents{};
    if (e.start && name) {
        std::lock_guard<std::mutex> lk(g_prof_mu);
        for (auto it = g_prof.rbegin(); it != g_prof.rend(); ++it)
            if (it->a == (hipEvent_t)e.start) {
                it->name = name;
                break;
            }
    }
    return e;
}
void prof_end(int token, void* stream) {
    if (token < 0) return;
    // no kernel took the events (the call returned before its launch): record them so that the pair is complete
    ProfEvents e = prof_take();
    if (e.start) {
        (void)hipEventRecord((hipEvent_t)e.start, (hipStream_t)stream);
        (void)hipEventRecord((hipEvent_t)e.stop, (hipStream_t)stream);
    }
}

}  // namespace tfh

using tfh::hip_check;
using tfh::set_error;

extern "C" {

int32_t tfh_profile_enable(int32_t on) {
    std::lock_guard<std::mutex> lk(tfh::g_prof_mu);
    for (auto& r : tfh::g_prof) {
        (void)hipEventSynchronize(r.b);
        tfh::g_prof_pool.push_back(r.a);
        tfh::g_prof_pool.push_back(r.b);
    }
    tfh::g_prof.clear();
    tfh::g_prof_on = on != 0;
    return TFH_OK;
}

int32_t tfh_profile_collect(int32_t kind, double* total_ms, int32_t* launches) {
    if (!total_ms || !launches) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    std::lock_guard<std::mutex> lk(tfh::g_prof_mu);
    double total = 0;
    int n = 0;
    std::vector<tfh::ProfRec> keep;
    for (auto& r : tfh::g_prof) {
        if (r.kind != kind) {
            keep.push_back(r);
            continue;
        }
        if (int32_t e = hip_check(hipEventSynchronize(r.b), "hipEventSynchronize")) return e;
        float ms = 0;
        if (int32_t e = hip_check(hipEventElapsedTime(&ms, r.a, r.b), "hipEventElapsedTime")) return e;
        total += ms;
        ++n;
        tfh::g_prof_pool.push_back(r.a);
        tfh::g_prof_pool.push_back(r.b);
    }
    tfh::g_prof.swap(keep);
    *total_ms = total;
    *launches = n;
    return TFH_OK;
}

int32_t tfh_profile_kernel(int32_t kind, int32_t index, char* name, size_t cap, double* total_ms, int32_t* launches) {
    if (!name || !cap || !total_ms || !launches || index < 0) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer or negative index");
    std::lock_guard<std::mutex> lk(tfh::g_prof_mu);
    std::vector<const char*> names;   // distinct labels of this kind in order of first launch (labels are unique pointers per kernel)
    for (auto& r : tfh::g_prof) {
        if (r.kind != kind) continue;
        bool seen = false;
        for (const char* n : names) seen = seen || std::string(n) == r.name;
        if (!seen) names.push_back(r.name);
    }
    name[0] = 0;
    *total_ms = 0;
    *launches = 0;
    if ((size_t)index >= names.size()) return TFH_OK;
    snprintf(name, cap, "%s", names[(size_t)index]);
    for (auto& r : tfh::g_prof) {
        if (r.kind != kind || std::string(r.name) != names[(size_t)index]) continue;
        if (int32_t e = hip_check(hipEventSynchronize(r.b), "hipEventSynchronize")) return e;
        float ms = 0;
        if (int32_t e = hip_check(hipEventElapsedTime(&ms, r.a, r.b), "hipEventElapsedTime")) return e;
        *total_ms += ms;
        ++*launches;
    }
    return TFH_OK;
}

const char* tfh_last_kernel(void) { return tfh::last_kernel(); }

int32_t tfh_release_workspaces(void) {
    std::lock_guard<std::mutex> lk(tfh::g_mu);
    tfh::g_table_epoch.fetch_add(1, std::memory_order_acq_rel);   // recorded launches that name cached tables are void from here on
    if (int32_t e = hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize")) return e;
    for (auto& kv : tfh::g_scratch) {
        auto& sc = kv.second;
        if (sc.ws && !sc.ws_pinned) {
            (void)hipFree(sc.ws);
            sc.ws = nullptr;
            sc.ws_bytes = 0;
        }
        for (auto it = sc.free_blocks.begin(); it != sc.free_blocks.end();) {
            if (sc.pinned_blocks.count(it->second)) {
                ++it;
                continue;
            }
            (void)hipFree(it->second);
            it = sc.free_blocks.erase(it);
        }
        for (auto it = sc.tables.begin(); it != sc.tables.end();) {
            if (it->second.pinned) {
                ++it;
                continue;
            }
            (void)hipFree(it->second.dev);
            sc.table_bytes -= it->second.bytes;
            it = sc.tables.erase(it);
        }
        tfh::free_bounce(sc);   // (the device is idle: no copy is using the staging buffers)
    }
    return TFH_OK;
}

int32_t tfh_device_count(int32_t* n) {
    if (!n) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    int c = 0;
    hipError_t e = hipGetDeviceCount(&c);
    if (e == hipErrorNoDevice) {
        *n = 0;
        (void)hipGetLastError();
        return TFH_OK;
    }
    if (int32_t s = hip_check(e, "hipGetDeviceCount")) return s;
    *n = c;
    return TFH_OK;
}

int32_t tfh_set_device(int32_t device_id) { return hip_check(hipSetDevice(device_id), "hipSetDevice"); }

int32_t tfh_preferred_compute_devices(int32_t space_kind, int64_t space_id, int32_t op_kind, tfh_compute_device* out,
                                      int32_t cap, int32_t* n) {
    // preferred_compute_devices(space, op_kind) (tenferro-device/src/lib.rs:92-105).  This library
    // computes on HIP devices only: GpuMemory{id} -> [Hip{id}] when that device exists.
    if (!n) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *n = 0;
    if (op_kind < TFH_KIND_CONTRACT || op_kind > TFH_KIND_ELEMENTWISE_MUL) return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown OpKind %d", op_kind);
    if (space_kind == TFH_SPACE_GPU_MEMORY) {
        int32_t count = 0;
        if (int32_t e = tfh_device_count(&count)) return e;
        if (space_id >= 0 && space_id < count) {
            if (out && cap > 0) {
                out[0].kind = TFH_DEVICE_HIP;
                out[0].device_id = (int32_t)space_id;
            }
            *n = 1;
            return TFH_OK;
        }
        return tfh::set_no_compatible_device(space_kind, space_id, op_kind);
    }
    if (space_kind == TFH_SPACE_MAIN_MEMORY) return tfh::set_no_compatible_device(space_kind, 0, op_kind);
    return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown memory space kind %d", space_kind);
}

int32_t tfh_malloc(size_t bytes, void** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    if (hipMalloc(out, bytes ? bytes : 1) == hipSuccess) return TFH_OK;
    (void)hipGetLastError();
    std::lock_guard<std::mutex> lk(tfh::g_mu);
    return tfh::malloc_or_release(out, bytes ? bytes : 1, nullptr, "hipMalloc");
}
int32_t tfh_free(void* ptr) { return hip_check(hipFree(ptr), "hipFree"); }
int32_t tfh_memcpy_h2d(void* dst, const void* src, size_t bytes, tfh_stream stream) {
    if (bytes == 0) return TFH_OK;
    if (!dst || !src) return set_error(TFH_ERR_INVALID_ARGUMENT, "null pointer");
    if (tfh::is_pinned_host(src) || tfh::capturing(stream))
        return hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream), "hipMemcpyAsync(h2d)");
    return tfh::staged_h2d(dst, src, bytes, stream);
}
int32_t tfh_memcpy_d2h(void* dst, const void* src, size_t bytes, tfh_stream stream) {
    if (bytes == 0) return TFH_OK;
    if (!dst || !src) return set_error(TFH_ERR_INVALID_ARGUMENT, "null pointer");
    if (tfh::is_pinned_host(dst) || tfh::capturing(stream))
        return hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync(d2h)");
    return tfh::staged_d2h(dst, src, bytes, stream);
}
int32_t tfh_host_malloc(size_t bytes, void** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    return hip_check(hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault), "hipHostMalloc");
}
int32_t tfh_host_free(void* ptr) { return hip_check(hipHostFree(ptr), "hipHostFree"); }
int32_t tfh_memcpy_d2d(void* dst, const void* src, size_t bytes, tfh_stream stream) {
    return hip_check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream), "hipMemcpyAsync(d2d)");
}

int32_t tfh_stream_create(tfh_stream* out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    hipStream_t s = nullptr;
    if (int32_t e = hip_check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate")) return e;
    *out = s;
    return TFH_OK;
}
// The stream's scratch goes with it: workspace, cached intermediates, offset tables and the pinned staging buffers are
// freed once the stream's work has finished, so that a later stream that happens to get the same handle value starts
// clean.  Buffers that were handed out during a graph capture stay alive (the graph may be replayed on another stream).
int32_t tfh_stream_destroy(tfh_stream s) {
    if (int32_t e = hip_check(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize")) return e;
    {
        std::lock_guard<std::mutex> lk(tfh::g_mu);
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess) {
            auto it = tfh::g_scratch.find({dev, (void*)s});
            if (it != tfh::g_scratch.end()) {
                auto& sc = it->second;
                if (!sc.tables.empty()) tfh::g_table_epoch.fetch_add(1, std::memory_order_acq_rel);
                if (sc.ws) {
                    if (sc.ws_pinned) tfh::g_orphans.push_back(sc.ws);
                    else (void)hipFree(sc.ws);
                }
                for (void* p : sc.retired) tfh::g_orphans.push_back(p);
                for (auto& fb : sc.free_blocks) {
                    if (sc.pinned_blocks.count(fb.second)) tfh::g_orphans.push_back(fb.second);
                    else (void)hipFree(fb.second);
                }
                for (auto& t : sc.tables) {
                    if (t.second.pinned) tfh::g_orphans.push_back(t.second.dev);
                    else (void)hipFree(t.second.dev);
                }
                tfh::free_bounce(sc);
                // (blocks still handed out belong to their holders: the entry stays until they are back)
                if (sc.live.empty()) tfh::g_scratch.erase(it);
                else {
                    sc.ws = nullptr; sc.ws_bytes = 0; sc.ws_pinned = false;
                    sc.retired.clear(); sc.free_blocks.clear(); sc.tables.clear(); sc.table_bytes = 0;
                }
            }
        } else {
            (void)hipGetLastError();
        }
    }
    return hip_check(hipStreamDestroy((hipStream_t)s), "hipStreamDestroy");
}
int32_t tfh_stream_synchronize(tfh_stream s) { return hip_check(hipStreamSynchronize((hipStream_t)s), "hipStreamSynchronize"); }

int32_t tfh_event_create(tfh_event* out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    hipEvent_t e = nullptr;
    if (int32_t s = hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate")) return s;
    *out = e;
    return TFH_OK;
}
int32_t tfh_event_destroy(tfh_event e) { return hip_check(hipEventDestroy((hipEvent_t)e), "hipEventDestroy"); }
int32_t tfh_event_record(tfh_event e, tfh_stream s) { return hip_check(hipEventRecord((hipEvent_t)e, (hipStream_t)s), "hipEventRecord"); }
int32_t tfh_event_synchronize(tfh_event e) { return hip_check(hipEventSynchronize((hipEvent_t)e), "hipEventSynchronize"); }
int32_t tfh_event_query(tfh_event e, int32_t* ready) {
    if (!ready) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    hipError_t r = hipEventQuery((hipEvent_t)e);
    if (r == hipSuccess) { *ready = 1; return TFH_OK; }
    if (r == hipErrorNotReady) { *ready = 0; (void)hipGetLastError(); return TFH_OK; }
    return hip_check(r, "hipEventQuery");
}
int32_t tfh_stream_wait_event(tfh_stream s, tfh_event e) {
    return hip_check(hipStreamWaitEvent((hipStream_t)s, (hipEvent_t)e, 0), "hipStreamWaitEvent");
}

}  // extern "C"
