/*
 * tenferro_hip.h -- C ABI of the MI355X (gfx950) backend for tenferro's tensor
 * primitives and einsum executor.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, never throws
 * and never aborts: it returns a tfh_status and leaves a description of the failure
 * in a thread-local slot read with tfh_last_error().  The scalar type crosses the
 * boundary as a run-time tag (tfh_dtype) because generics cannot; a Rust binding
 * monomorphises back (`impl TensorPrims<Standard> for HipBackend`).
 *
 * Threads: every entry point may be called from any thread, and calls that enqueue on
 * DIFFERENT streams may run concurrently.  Each stream owns scratch memory (offset tables,
 * split-K partials, einsum intermediates) that the kernels of successive calls reuse in
 * stream order, so calls that enqueue on the SAME stream must not overlap in time: the
 * caller serialises them, as it would the launches themselves.
 *
 * Reference interfaces replaced (paths relative to the tenferro-rs workspace):
 *   tenferro-prims/src/lib.rs:278-340   trait TensorPrims<A> { plan, execute, has_extension_for }
 *   tenferro-prims/src/lib.rs:152-245   enum PrimDescriptor
 *   tenferro-prims/src/lib.rs:100-128   enum ReduceOp, enum Extension
 *   tenferro-einsum/src/lib.rs:239-356  Subscripts, ContractionTree
 *   tenferro-einsum/src/lib.rs:393-621  einsum* entry points
 *   tenferro-tensor/src/lib.rs:133-181  DataBuffer / Tensor storage (device buffer, event)
 *   tenferro-tensor/src/lib.rs:622-658  Tensor::conj / into_conj
 *   tenferro-device/src/lib.rs:30-162   LogicalMemorySpace, ComputeDevice, OpKind, Error
 */
#ifndef TENFERRO_HIP_H
#define TENFERRO_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TFH_MAX_RANK 16

/* ---- status codes: one per variant of tenferro_device::Error (tenferro-device/src/lib.rs:108-159) */
typedef enum tfh_status {
    TFH_OK = 0,
    TFH_ERR_SHAPE_MISMATCH = 1,        /* Error::ShapeMismatch { expected, got }           :111-117 */
    TFH_ERR_RANK_MISMATCH = 2,         /* Error::RankMismatch { expected, got }            :119-126 */
    TFH_ERR_DEVICE = 3,                /* Error::DeviceError(String)                       :128-130 */
    TFH_ERR_NO_COMPATIBLE_DEVICE = 4,  /* Error::NoCompatibleComputeDevice { space, op }   :132-140 */
    TFH_ERR_CROSS_MEMORY_SPACE = 5,    /* Error::CrossMemorySpaceOperation { left, right } :142-150 */
    TFH_ERR_INVALID_ARGUMENT = 6,      /* Error::InvalidArgument(String)                   :152-154 */
    TFH_ERR_STRIDED = 7                /* Error::Strided(StridedError)                     :156-158 */
} tfh_status;

/* Payload of the last failure on the calling thread: what a binding needs to rebuild the Error variant.
 *   ShapeMismatch              expected[0..n_expected), got[0..n_got): the two shapes
 *   RankMismatch               expected[0], got[0]: the two ranks (n_expected = n_got = 1)
 *   NoCompatibleComputeDevice  expected[0..2) = the memory space as (tfh_space_kind, space id), got[0] = the tfh_op_kind
 *   CrossMemorySpaceOperation  expected[0..2) = the left space, got[0..2) = the right space, each (tfh_space_kind, id);
 *                              never returned by this library, whose views are bare device pointers: the binding,
 *                              which knows where its tensors live, raises it before calling (the layout is fixed
 *                              here so that every binding decodes status 5 the same way)
 *   DeviceError, InvalidArgument, Strided   message only */
typedef struct tfh_error_info {
    int32_t status;                    /* tfh_status of the failing call */
    int32_t n_expected;
    int32_t n_got;
    int32_t reserved;
    int64_t expected[TFH_MAX_RANK];
    int64_t got[TFH_MAX_RANK];
    char message[512];                 /* NUL-terminated, formatted like the Rust Display impl */
} tfh_error_info;

/* Copies the calling thread's last error into *out (status TFH_OK if none). */
void tfh_last_error(tfh_error_info* out);
const char* tfh_status_name(int32_t status);
const char* tfh_version(void);

/* ---- scalar types: the Standard-algebra set (tenferro-algebra/src/lib.rs:58-72) */
typedef enum tfh_dtype {
    TFH_F32 = 0,
    TFH_F64 = 1,
    TFH_C64 = 2,   /* Complex32: interleaved (re, im) f32 */
    TFH_C128 = 3   /* Complex64: interleaved (re, im) f64 */
} tfh_dtype;
size_t tfh_dtype_size(int32_t dtype);

/* ---- strided view: the StridedView / StridedViewMut contract with a DEVICE base pointer.
 * dims as usize, strides as isize "in units of T", offset as isize
 * (tenferro-tensor/src/lib.rs:169-171, 219-221).  Element (i0, i1, ...) lives at
 * base + (offset + sum_d i_d * strides[d]) * sizeof(T).  Zero strides (broadcast,
 * tenferro-tensor/src/lib.rs:506-516) and negative strides are legal for inputs. */
typedef struct tfh_view {
    void* base;
    int32_t rank;
    int32_t flags;        /* TFH_VIEW_* bits; 0 for a plain view */
    int64_t offset;
    int64_t dims[TFH_MAX_RANK];
    int64_t strides[TFH_MAX_RANK];
} tfh_view;

/* TFH_VIEW_CONJ on an INPUT view of a complex dtype: the operation reads conj(element) instead of the element, without
 * a conjugated copy -- the lazy form of Tensor::conj (tenferro-tensor/src/lib.rs:622-658), an addition to the
 * reference's views.  Honoured by Contract, BatchedGemm, Permute and by the operands of tfh_einsum_execute: the
 * contraction kernels flip the sign of the imaginary part while they stage the operand.  Ignored for real dtypes; any
 * other operation, an output view and a grouped plan reject it with TFH_ERR_INVALID_ARGUMENT. */
#define TFH_VIEW_CONJ 1

/* ---- operation descriptor: PrimDescriptor (tenferro-prims/src/lib.rs:152-245) */
typedef enum tfh_op {
    TFH_OP_BATCHED_GEMM = 0,    /* :156-168  C[batch,m,n] = a*A[batch,m,k]*B[batch,k,n] + b*C */
    TFH_OP_REDUCE = 1,          /* :170-180  C[modes_c] = a*reduce_op(A[modes_a]) + b*C       */
    TFH_OP_TRACE = 2,           /* :182-192  sum over the diagonal of each paired mode        */
    TFH_OP_PERMUTE = 3,         /* :194-202  B[modes_b] = a*A[modes_a]   (modes_c holds modes_b) */
    TFH_OP_ANTI_TRACE = 4,      /* :204-212  scatter-add to the diagonal                      */
    TFH_OP_ANTI_DIAG = 5,       /* :214-222  write to the diagonal                            */
    TFH_OP_CONTRACT = 6,        /* :227-239  C[modes_c] = a*contract(A[modes_a],B[modes_b]) + b*C */
    TFH_OP_ELEMENTWISE_MUL = 7  /* :241-244  C = a*A.*B + b*C, same-shape views               */
} tfh_op;

typedef enum tfh_reduce_op { TFH_REDUCE_SUM = 0, TFH_REDUCE_MAX = 1, TFH_REDUCE_MIN = 2 } tfh_reduce_op; /* :100-107 */
typedef enum tfh_extension { TFH_EXT_CONTRACT = 0, TFH_EXT_ELEMENTWISE_MUL = 1 } tfh_extension;          /* :123-128 */

typedef struct tfh_desc {
    int32_t op;                  /* tfh_op */
    int32_t reduce_op;           /* tfh_reduce_op, REDUCE only */
    /* BatchedGemm fields */
    const int64_t* batch_dims;
    int32_t n_batch_dims;
    int32_t reserved;
    int64_t m, n, k;
    /* mode labels (u32, cuTENSOR convention, tenferro-prims/src/lib.rs:136-138) */
    const uint32_t* modes_a; int32_t n_modes_a;
    const uint32_t* modes_b; int32_t n_modes_b;   /* Contract only (second input) */
    const uint32_t* modes_c; int32_t n_modes_c;   /* output modes (Permute: modes_b of the reference) */
    /* Trace / AntiTrace / AntiDiag: n_pairs pairs, flattened (i0, j0, i1, j1, ...) */
    const uint32_t* paired; int32_t n_pairs;
} tfh_desc;

/* ---- TensorPrims<Standard> for the Hip backend ------------------------------------------- */

typedef struct tfh_plan tfh_plan;   /* opaque; immutable after creation; shareable across threads */
typedef void* tfh_stream;           /* hipStream_t; NULL = the null stream */
typedef void* tfh_event;            /* hipEvent_t */

/* TensorPrims::has_extension_for::<T>(ext)  (tenferro-prims/src/lib.rs:322-339). Returns 1 or 0. */
int32_t tfh_has_extension(int32_t dtype, int32_t ext);

/* TensorPrims::plan::<T>(desc, shapes)  (tenferro-prims/src/lib.rs:282-298).
 * shapes[i] has ranks[i] entries; inputs first, then the output (:284-286).
 * Validates the descriptor against the shapes; touches no device. */
int32_t tfh_plan_create(int32_t dtype, const tfh_desc* desc,
                        const int64_t* const* shapes, const int32_t* ranks, int32_t n_tensors,
                        tfh_plan** out);
void tfh_plan_destroy(tfh_plan* plan);

/* One-line description of a plan: operation, dtype, and -- for a Contract / BatchedGemm plan that has been executed -- the
 * kernels of the routes it keeps (one per set of view strides it has seen, see tfh_plan_cache_stats). */
int32_t tfh_plan_describe(const tfh_plan* plan, char* buf, size_t cap);
/* "The plan pre-computes kernel selection" (tenferro-prims/src/lib.rs:8, :284): what the route of a contraction depends on
 * besides the extents -- the views' strides -- only shows at execute, so a Contract / BatchedGemm plan keeps the routed
 * launch of the first execute with each set of strides (up to eight) and later executes with the same strides enqueue it
 * again on their buffers without routing.  This reads the plan's counters: executes that found their route, executes
 * that had to route, routes kept (any pointer may be null; all zero for other operations). */
int32_t tfh_plan_cache_stats(const tfh_plan* plan, int64_t* hits, int64_t* misses, int32_t* entries);

/* TensorPrims::execute(plan, alpha, inputs, beta, output)  (tenferro-prims/src/lib.rs:300-320).
 * output = alpha*op(inputs) + beta*output; beta == 0 overwrites without reading the output.
 * alpha/beta point at one host scalar of the plan's dtype.  Kernels are enqueued on `stream`;
 * the call does not wait for them. */
int32_t tfh_execute(const tfh_plan* plan, const void* alpha,
                    const tfh_view* inputs, int32_t n_inputs,
                    const void* beta, tfh_view* output, tfh_stream stream);

/* Grouped (variable-size) execution: n_groups independent problems that share one descriptor
 * but not their extents, as the blocks of a block-sparse contraction do.  The reference
 * protocol has no grouped descriptor (BatchedGemm is uniform-size, tenferro-prims/src/lib.rs:
 * 159-168); this is an additive extension that leaves TensorPrims untouched.
 * shapes holds n_groups*n_tensors pointers, group-major (inputs first, then output). */
int32_t tfh_plan_create_grouped(int32_t dtype, const tfh_desc* desc, int32_t n_groups,
                                const int64_t* const* shapes, const int32_t* ranks, int32_t n_tensors,
                                tfh_plan** out);
/* inputs: n_groups*n_inputs views, group-major; outputs: n_groups views.  One launch of the contraction; the
 * problems' pointers, extents and strides are written to the device by small launches in front of it, and kept with
 * the plan (up to eight sets per device), so that a call whose views equal those of an earlier call skips them.
 * The plan must outlive the work enqueued through it (as its tile maps always had to). */
int32_t tfh_execute_grouped(const tfh_plan* plan, const void* alpha,
                            const tfh_view* inputs, int32_t n_inputs,
                            const void* beta, tfh_view* outputs, tfh_stream stream);

/* tfh_execute for callers that cannot allocate device memory.  No counterpart in the reference: it is for code
 * under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc.  Same arguments, same kernels
 * and same results as tfh_execute, but the device scratch of the call (offset tables, split-K partials, partial sums
 * of a split reduction, a packed copy of an operand) comes from one fixed array of TFH_STATIC_SCRATCH_BYTES that is
 * part of the library's code object on every device it runs on; the call allocates and frees nothing on the device.
 * A call that needs more scratch than that fails with TFH_ERR_INVALID_ARGUMENT and a message that gives the
 * amounts (kernels that precede the oversized request may already have been enqueued; the output is then
 * unspecified).  All calls on one device share the array: calls that overlap in time on one device, on any
 * streams or threads, race on it -- order them on one stream or with events.  Grouped plans are not taken. */
#define TFH_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
size_t tfh_static_scratch_bytes(void);
int32_t tfh_execute_static(const tfh_plan* plan, const void* alpha,
                           const tfh_view* inputs, int32_t n_inputs,
                           const void* beta, tfh_view* output, tfh_stream stream);

/* Tensor::conj / into_conj (tenferro-tensor/src/lib.rs:622-658): out = conj(in) elementwise,
 * same dims; a plain copy for real dtypes.  in and out may be the same view (into_conj). */
int32_t tfh_conj(int32_t dtype, const tfh_view* in, tfh_view* out, tfh_stream stream);
/* Tensor::zeros / ones (tenferro-tensor/src/lib.rs:336-347) on device memory: fill a view with
 * one host scalar of `dtype`. */
int32_t tfh_fill(int32_t dtype, const void* value, tfh_view* out, tfh_stream stream);

/* ---- einsum front end and executor --------------------------------------------------------- */

typedef struct tfh_subscripts tfh_subscripts;   /* Subscripts (tenferro-einsum/src/lib.rs:239-245) */
typedef struct tfh_tree tfh_tree;               /* ContractionTree (:297-300) */

/* Subscripts::new(inputs, output) (:253-258).  labels holds the concatenated input labels. */
int32_t tfh_subscripts_new(const uint32_t* labels, const int32_t* ranks, int32_t n_inputs,
                           const uint32_t* output, int32_t n_output, tfh_subscripts** out);
/* Subscripts::parse(notation) (:260-283): a-zA-Z labels, ',' and '->', parentheses for an
 * explicit pairwise order.  Malformed notation -> TFH_ERR_INVALID_ARGUMENT. */
int32_t tfh_subscripts_parse(const char* notation, tfh_subscripts** out);
void tfh_subscripts_destroy(tfh_subscripts* s);
int32_t tfh_subscripts_n_inputs(const tfh_subscripts* s);
int32_t tfh_subscripts_input_rank(const tfh_subscripts* s, int32_t i);
/* Copies the labels of input i (or of the output when i == -1) into out[cap]; returns the rank. */
int32_t tfh_subscripts_labels(const tfh_subscripts* s, int32_t i, uint32_t* out, int32_t cap);
/* The parenthesisation as written, operands by index: "ij,(jk,kl)->il" gives "0,(1,2)". */
int32_t tfh_subscripts_nesting(const tfh_subscripts* s, char* buf, size_t cap);

/* ContractionTree::optimize(subscripts, shapes) (:303-318): minimum total operation count;
 * exhaustive over subsets up to 12 operands, greedy beyond.  If the subscripts carry
 * parentheses the order they spell is used instead. */
int32_t tfh_tree_optimize(const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks,
                          int32_t n_inputs, tfh_tree** out);
/* ContractionTree::from_pairs(subscripts, shapes, pairs) (:320-355): intermediates are numbered
 * from n_inputs upward.  pairs holds 2*n_pairs operand indices. */
int32_t tfh_tree_from_pairs(const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks,
                            int32_t n_inputs, const int32_t* pairs, int32_t n_pairs, tfh_tree** out);
void tfh_tree_destroy(tfh_tree* t);
/* The same tree as tfh_tree_optimize, from a process-wide cache keyed on the subscripts (labels, grouping) and the
 * shapes: the string and allocating forms of einsum (tenferro-einsum/src/lib.rs:393-434, :541-582) optimise the same
 * network on every call, which costs 5 us for two operands and milliseconds for eight.  The tree is shared and
 * immutable; release it with tfh_tree_destroy like any other (trees are reference counted, so one that the cache has
 * dropped stays valid for its holders).  At most 512 networks are kept, least recently used dropped first. */
int32_t tfh_tree_optimize_cached(const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks,
                                 int32_t n_inputs, tfh_tree** out);
int32_t tfh_tree_cache_stats(int64_t* hits, int64_t* misses, int64_t* entries);   /* any pointer may be null */
int32_t tfh_tree_cache_clear(void);
int32_t tfh_tree_n_inputs(const tfh_tree* t);
int32_t tfh_tree_n_steps(const tfh_tree* t);
/* Step i contracts operands (lhs, rhs) into intermediate n_inputs + i. */
int32_t tfh_tree_step(const tfh_tree* t, int32_t i, int32_t* lhs, int32_t* rhs);
/* Labels and extents of a node (input, intermediate or the final result = n_inputs+n_steps-1,
 * whose order is the requested output order).  Returns the rank. */
int32_t tfh_tree_node(const tfh_tree* t, int32_t node, uint32_t* labels, int64_t* dims, int32_t cap);
int32_t tfh_tree_output_rank(const tfh_tree* t);
int32_t tfh_tree_output_dims(const tfh_tree* t, int64_t* dims, int32_t cap);
/* Multiply-add count of the tree (one per scalar multiply-add; a complex one counts once) and
 * the element count of the largest intermediate. */
double tfh_tree_mac_count(const tfh_tree* t);
double tfh_tree_peak_intermediate(const tfh_tree* t);

/* einsum_with_plan_into(tree, operands, alpha, beta, output) (tenferro-einsum/src/lib.rs:584-621):
 * output = alpha*einsum(operands) + beta*output.  All kernels of the tree are enqueued on
 * `stream`; intermediates stay in device memory; the host never waits.  The allocating and
 * string/subscript variants (:393-498, :541-582) are this call behind tfh_subscripts_parse,
 * tfh_tree_optimize and an output buffer sized with tfh_tree_output_dims.
 * donate_mask: bit i set = operand i's buffer may be overwritten (the *_owned variants, :436-498):
 * a dense operand that overlaps no other operand nor the output may hold an intermediate of a
 * step later than the one that reads it.  Its contents after the call are unspecified. */
int32_t tfh_einsum_execute(int32_t dtype, const tfh_tree* tree,
                           const tfh_view* operands, int32_t n_operands,
                           const void* alpha, const void* beta, tfh_view* output,
                           uint64_t donate_mask, tfh_stream stream);

/* ---- device, memory, streams, events ------------------------------------------------------- */

/* OpKind (tenferro-device/src/lib.rs:77-90) */
typedef enum tfh_op_kind {
    TFH_KIND_CONTRACT = 0, TFH_KIND_BATCHED_GEMM = 1, TFH_KIND_REDUCE = 2,
    TFH_KIND_TRACE = 3, TFH_KIND_PERMUTE = 4, TFH_KIND_ELEMENTWISE_MUL = 5
} tfh_op_kind;
typedef enum tfh_space_kind { TFH_SPACE_MAIN_MEMORY = 0, TFH_SPACE_GPU_MEMORY = 1 } tfh_space_kind;   /* :30-38 */
typedef enum tfh_device_kind { TFH_DEVICE_CPU = 0, TFH_DEVICE_CUDA = 1, TFH_DEVICE_HIP = 2 } tfh_device_kind; /* :46-62 */
typedef struct tfh_compute_device { int32_t kind; int32_t device_id; } tfh_compute_device;

/* preferred_compute_devices(space, op_kind) (tenferro-device/src/lib.rs:92-105): GpuMemory{n}
 * -> [Hip{n}] when device n exists; MainMemory or an unknown space -> NoCompatibleComputeDevice
 * (this library computes on HIP devices only).  Writes up to cap devices, count in *n. */
int32_t tfh_preferred_compute_devices(int32_t space_kind, int64_t space_id, int32_t op_kind,
                                      tfh_compute_device* out, int32_t cap, int32_t* n);
/* Display for ComputeDevice (tenferro-device/src/lib.rs:64-72): "cpu:0", "cuda:1", "hip:0". */
int32_t tfh_compute_device_format(int32_t kind, int64_t device_id, char* buf, size_t cap);

int32_t tfh_device_count(int32_t* n);
int32_t tfh_set_device(int32_t device_id);

/* DataBuffer::Hip storage (tenferro-tensor/src/lib.rs:133-137). */
int32_t tfh_malloc(size_t bytes, void** out);
int32_t tfh_free(void* ptr);
/* Tensor::to_memory_space_async (tenferro-tensor/src/lib.rs:660-671).  Host memory from tfh_host_malloc (page-locked)
 * is copied by the copy engine directly and the call returns at once; the transfer is complete when work enqueued on
 * `stream` after it runs (record an event).  Ordinary (pageable) host memory goes through two 16 MiB pinned staging
 * buffers of the stream, in chunks, the host filling or emptying one while the engine works on the other: the call
 * returns when the host side is done -- host-to-device: the source may be reused, the last chunk is on its way in
 * stream order; device-to-host: the data is in `dst`.  Either way the transfer runs beside kernels of other streams. */
int32_t tfh_memcpy_h2d(void* dst, const void* src, size_t bytes, tfh_stream stream);
int32_t tfh_memcpy_d2h(void* dst, const void* src, size_t bytes, tfh_stream stream);
int32_t tfh_memcpy_d2d(void* dst, const void* src, size_t bytes, tfh_stream stream);
/* Page-locked host memory for transfers that return immediately (no counterpart in the reference, whose host tensors
 * are ordinary Vec<T>; a MainMemory tensor that is meant to move may be allocated here). */
int32_t tfh_host_malloc(size_t bytes, void** out);
int32_t tfh_host_free(void* ptr);

int32_t tfh_stream_create(tfh_stream* out);
int32_t tfh_stream_destroy(tfh_stream s);
int32_t tfh_stream_synchronize(tfh_stream s);

/* CompletionEvent (tenferro-tensor/src/lib.rs:301-309); Tensor::wait / is_ready (:677-713). */
int32_t tfh_event_create(tfh_event* out);
int32_t tfh_event_destroy(tfh_event e);
int32_t tfh_event_record(tfh_event e, tfh_stream s);
int32_t tfh_event_synchronize(tfh_event e);             /* Tensor::wait */
int32_t tfh_event_query(tfh_event e, int32_t* ready);   /* Tensor::is_ready */
int32_t tfh_stream_wait_event(tfh_stream s, tfh_event e);  /* chaining without a host wait (tenferro-einsum/src/lib.rs:146-177) */

/* Measurement aid (no counterpart in the reference): while enabled, the dominant kernel of every
 * contraction (kind 0), copy/permute (kind 1) and reduction (kind 2) launch is bracketed by HIP events
 * on its own stream.  tfh_profile_collect waits for them and returns the summed duration and the
 * launch count of one kind since the last enable, then forgets those records. */
int32_t tfh_profile_enable(int32_t on);
int32_t tfh_profile_collect(int32_t kind, double* total_ms, int32_t* launches);
/* The same records by kernel, before tfh_profile_collect forgets them: the index-th distinct kernel (in order of its
 * first launch) among the records of one kind, its label as tfh_last_kernel spells it, the summed duration and
 * the number of its launches.  *launches == 0 and an empty name: index is past the last kernel. */
int32_t tfh_profile_kernel(int32_t kind, int32_t index, char* name, size_t cap, double* total_ms, int32_t* launches);

/* Diagnostic, no counterpart in the reference: the name, in parentheses and with its template arguments as
 * instantiated ("(gemm128_kernel<double, true, false, true, 1, 1, 128>)", what a kernel trace shows without namespaces
 * and parameter list), of the dominant kernel most recently launched by the calling thread, "" before the first one.
 * Tests use it to check which kernel a call was routed to. */
const char* tfh_last_kernel(void);

/* Releases the cached workspace, intermediate buffers and offset tables of every stream (after a synchronize).
 * Buffers that were handed out while their stream was being captured into a HIP graph are part of that graph and are
 * passed over, here and whenever the library frees or regrows a cache: they stay until the process ends. */
int32_t tfh_release_workspaces(void);

#ifdef __cplusplus
}
#endif
#endif /* TENFERRO_HIP_H */
