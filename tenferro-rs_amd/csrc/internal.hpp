// internal.hpp -- types shared by the host side of the backend (not part of the C ABI).
#pragma once
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../../include/tenferro_hip.h"

namespace tfh {

// ---- error reporting -----------------------------------------------------------------------------
// Each failing call records one of tenferro_device::Error's variants (tenferro-device/src/lib.rs:108-159)
// in a thread-local slot and returns its status code.
int32_t set_error(int32_t status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int32_t set_shape_mismatch(const int64_t* expected, int n_expected, const int64_t* got, int n_got);
int32_t set_rank_mismatch(int64_t expected, int64_t got);
int32_t set_no_compatible_device(int32_t space_kind, int64_t space_id, int32_t op_kind);
void clear_error();

inline bool is_complex(int dt) { return dt == TFH_C64 || dt == TFH_C128; }
inline bool is_double(int dt) { return dt == TFH_F64 || dt == TFH_C128; }
inline size_t dtype_size(int dt) {
    switch (dt) {
        case TFH_F32: return 4;
        case TFH_F64: return 8;
        case TFH_C64: return 8;
        case TFH_C128: return 16;
        default: return 0;
    }
}
// Host scalar of any dtype widened to (re, im) doubles.
struct Scalar {
    double re = 0, im = 0;
    bool is_zero() const { return re == 0 && im == 0; }
    bool is_one() const { return re == 1 && im == 0; }
};
inline Scalar load_scalar(int dt, const void* p) {
    Scalar s;
    if (is_double(dt)) {
        s.re = ((const double*)p)[0];
        if (is_complex(dt)) s.im = ((const double*)p)[1];
    } else {
        s.re = ((const float*)p)[0];
        if (is_complex(dt)) s.im = ((const float*)p)[1];
    }
    return s;
}

// One loop axis with an element stride per tensor slot (0 = the tensor does not carry it).
struct Axis {
    int64_t n;
    int64_t s[3];
    uint32_t label;
};

// ---- plan ----------------------------------------------------------------------------------------
struct GroupedState;  // device tables of a grouped plan (gemm.cpp)
struct ContractCache;  // routed launches of earlier calls of a Contract / BatchedGemm plan (contract_cache.cpp)
}  // namespace tfh

struct tfh_plan {
    int32_t dtype = 0;
    int32_t op = 0;
    int32_t reduce_op = 0;
    std::vector<uint32_t> modes_a, modes_b, modes_c;
    std::vector<std::pair<uint32_t, uint32_t>> pairs;
    int32_t n_inputs = 0;
    // expected shapes, inputs first then output; for a grouped plan n_groups*(n_inputs+1) entries
    std::vector<std::vector<int64_t>> shapes;
    int32_t n_groups = 0;  // 0 = not grouped
    tfh::GroupedState* grouped = nullptr;
    // Kernel selection is part of the plan (tenferro-prims/src/lib.rs:8, :284): the first execute with a given set of view
    // strides routes the contraction and keeps the routed launch here; later executes with the same strides only patch
    // the buffer addresses and scalars into it.  Guarded by its own lock: the plan stays shareable between threads.
    tfh::ContractCache* contract_cache = nullptr;
    ~tfh_plan();
};

namespace tfh {

// Validation + normalisation of a descriptor: BatchedGemm is rewritten as a Contract over synthetic
// labels; returns TFH_OK or records an error.
int32_t make_plan(int32_t dtype, const tfh_desc* desc, const int64_t* const* shapes, const int32_t* ranks,
                  int32_t n_tensors, tfh_plan& plan);
// Whether `stream` is recording a graph (nothing may be allocated or synchronised then).
bool stream_is_capturing(void* stream);
int32_t check_view_against(const std::vector<int64_t>& shape, const tfh_view& v, const char* what);

// Mode classification of a binary contraction (tenferro-prims/src/lib.rs:136-138).
struct ContractAxes {
    std::vector<Axis> batch, M, N, K;  // s[0]=A, s[1]=B, s[2]=C
};
int32_t classify_contract(const std::vector<uint32_t>& ma, const int64_t* dims_a, const int64_t* str_a,
                          const std::vector<uint32_t>& mb, const int64_t* dims_b, const int64_t* str_b,
                          const std::vector<uint32_t>& mc, const int64_t* dims_c, const int64_t* str_c,
                          ContractAxes& out);
// C = alpha * A * B + beta * C for a long operand against a small one (at most 64 real rows, 64 KB) that the
// register-resident streaming kernel does not take; true when it launched (k_gemm_thin.hip).
bool try_thin_stream(int dtype, const void* a, const void* b, void* c, const struct ContractAxes& ax, Scalar alpha, Scalar beta,
                     void* stream, bool conj_a, bool conj_b, int32_t& status);
// Drops extent-1 axes and merges neighbours that are contiguous in every slot in [0, nslots).
// Order is preserved (axis i+1 is "inside" axis i when they merge).
void fuse_axes(std::vector<Axis>& ax, int nslots);

// ---- kernel launchers (each enqueues on `stream`, returns a tfh_status) ----------------------------
// B = alpha*op(A) + beta*B over axes (s[0] = in stride, s[1] = out stride); op = conj if `conj`.
int32_t launch_copy(int dtype, const void* in, void* out, std::vector<Axis> axes, Scalar alpha, Scalar beta,
                    bool conj, void* stream);
// out = value over axes (s[0] = out stride)
int32_t launch_fill(int dtype, void* out, std::vector<Axis> axes, Scalar value, void* stream);
// C = alpha*A.*B + beta*C over axes (s[0]=A, s[1]=B, s[2]=C)
int32_t launch_emul(int dtype, const void* a, const void* b, void* c, std::vector<Axis> axes, Scalar alpha,
                    Scalar beta, void* stream);
// C[kept] = alpha*reduce(A[kept, red]) + beta*C ; kept: s[0]=A, s[1]=C ; red: s[0]=A
int32_t launch_reduce(int dtype, const void* a, void* c, std::vector<Axis> kept, std::vector<Axis> red, int reduce_op,
                      Scalar alpha, Scalar beta, void* stream);
// The general (any extents, any strides) reduction kernel; with b != nullptr the reduced quantity is the product A*B of
// two operands read at the same coordinates (sum only).  Axis slots here: 0 = A, 1 = C, 2 = B.
int32_t launch_reduce_general(int dtype, const void* a, const void* b, void* c, std::vector<Axis> kept, std::vector<Axis> red,
                              int reduce_op, Scalar alpha, Scalar beta, void* stream);
// What a contraction's launcher leaves behind for a repeated call: the routed launch (kernel, tile and split choice,
// operand exchange, table handles) with the buffer addresses and scalars taken out.  Defined by the launcher.
struct ContractRecord {
    std::string label;   // the kernel the route ends in, as tfh_last_kernel names it
    virtual ~ContractRecord() = default;
};
// C = alpha*A*B + beta*C over classified axes
// conj: bit 0 = conj(A), bit 1 = conj(B) (see k_gemm.hip)
// record: when non-null and the route is one that can be enqueued again without routing (no operand pack, no per-call
// table build), *record receives it.
int32_t launch_contract(int dtype, const void* a, const void* b, void* c, ContractAxes axes, Scalar alpha,
                        Scalar beta, void* stream, int conj = 0, std::shared_ptr<ContractRecord>* record = nullptr);
// Enqueues a recorded launch on new buffers (a, b: the first and second input as the caller passes them).  Returns false
// when the record no longer applies (the offset tables it names were released, another device is current): the caller
// routes the call again.
bool replay_contract(const ContractRecord& rec, int dtype, const void* a, const void* b, void* c, Scalar alpha, Scalar beta,
                     void* stream, int32_t& status);
// A contraction through a cache of routed launches (null: no cache).  The key is everything the route depends on besides
// the extents, which are fixed where the cache lives (a plan, a step of an einsum tree): the element type (a tree serves
// every type), the three views' strides, the 16-byte alignment classes of their addresses, the conj flags, whether beta
// is zero, the stream.
ContractCache* contract_cache_create();
void contract_cache_destroy(ContractCache* c);
void contract_cache_stats(const ContractCache* c, int64_t* hits, int64_t* misses, int32_t* entries);
// "<kernel label>; <kernel label>; ..." of the routes kept, oldest first (empty: none yet).
std::string contract_cache_routes(const ContractCache* c);
int32_t execute_contract(ContractCache* cache, int dtype, const std::vector<uint32_t>& ma, const int64_t* dims_a, const int64_t* str_a,
                         const void* a, const std::vector<uint32_t>& mb, const int64_t* dims_b, const int64_t* str_b, const void* b,
                         const std::vector<uint32_t>& mc, const int64_t* dims_c, const int64_t* str_c, void* c, Scalar alpha,
                         Scalar beta, void* stream, int conj);
// A tiny operator (<= 8 free and <= 8 contracted indices) applied to a long tensor: the streaming kernel of
// k_gemm_tiny.hip.  Returns false when the shape is not one it takes; true when it launched (status holds the outcome).
bool try_tiny_operator(int dtype, const void* a, const void* b, void* c, const ContractAxes& ax, Scalar alpha, Scalar beta,
                       void* stream, int32_t& status);
// Matrix-vector-like contractions (one free group empty): the streaming product-reduction kernel of k_dot.hip.  Returns
// false when the shape is not one it tiles; true when it launched (status holds the outcome).  Axis strides: A, B, C.
bool try_dot(int dtype, const void* a, const void* b, void* c, std::vector<Axis> kept, std::vector<Axis> red, Scalar alpha,
             Scalar beta, void* stream, int32_t& status);
// Counts the releases of cached offset tables (tfh_release_workspaces, a destroyed stream, the out-of-memory path): a
// recorded launch that names such tables is valid only while the count stands where it stood when the record was made.
uint64_t table_epoch();
int32_t grouped_plan_init(tfh_plan& plan);
int32_t launch_grouped(const tfh_plan& plan, Scalar alpha, const tfh_view* inputs, Scalar beta, tfh_view* outputs,
                       void* stream);
void grouped_state_destroy(GroupedState* g);

// ---- per-stream scratch memory ----------------------------------------------------------------------
// Workspace: one growing buffer per stream; kernels on a stream are ordered, so successive calls
// reuse it.  Valid until the next workspace() call on the same stream.
int32_t workspace(void* stream, size_t bytes, void** out);
// Offset tables of a contraction depend only on the fused dims and strides (`key`): the first call on a stream
// builds them with a kernel into a block that later calls on that stream reuse without a launch (stream order
// makes them ready).  *tables == nullptr: no cached block (cache full, stream being captured, entry being built by
// another thread) -- build them in the workspace.  *fresh: the caller fills the block, then calls commit.
int32_t table_cache_get(void* stream, const std::string& key, size_t bytes, void** tables, bool* fresh);
void table_cache_commit(void* stream, const std::string& key);
// Intermediates of an einsum tree: stream-ordered cached allocations (free returns the block to the
// stream's cache; reuse on the same stream needs no synchronisation).
int32_t pool_alloc(void* stream, size_t bytes, void** out);
void pool_free(void* stream, void* ptr);
// Between arena_begin() and arena_end() on one host thread, workspace() and pool_alloc() hand out consecutive pieces of
// the given device region instead of allocating (an error once it is used up), pool_free() does nothing and the table
// cache is bypassed.
void arena_begin(void* base, size_t bytes);
void arena_end();
int32_t hip_check(int err, const char* what);
// Event bracket around a dominant kernel while profiling is enabled (runtime.cpp); -1 when disabled.
enum { PROF_CONTRACT = 0, PROF_COPY = 1, PROF_REDUCE = 2 };
int prof_begin(int kind, void* stream);
// Remembers, per host thread, the source-level name of the dominant kernel launched last (tfh_last_kernel).
void note_kernel(const char* name);
void prof_end(int token, void* stream);
// The dominant kernel's launch takes the pair of events prof_begin() prepared on this thread (null when profiling is
// off): launched with them, the events carry the dispatch's own begin and end timestamps, so their difference is the
// kernel's duration as a kernel trace reports it, without the launch overhead two recorded events would add.
struct ProfEvents {
    void* start = nullptr;
    void* stop = nullptr;
};
// `name`: the label of the kernel that takes them, kept with the record (tfh_profile_kernel).
ProfEvents prof_take(const char* name = nullptr);

// Byte pointer of a view's element 0.
inline char* view_ptr(const tfh_view& v, int dtype) { return (char*)v.base + v.offset * (int64_t)dtype_size(dtype); }

}  // namespace tfh
