//! Raw FFI declarations of `libtenferro_hip.so`: one item per declaration of `include/tenferro_hip.h`, in the
//! header's order, with the header's argument names.  Nothing here is safe to call directly; the `tenferro-hip` crate
//! wraps these in the reference's own types (`HipBuffer`, `HipPlan`, `impl TensorPrims<Standard> for HipBackend`,
//! `CompletionEvent`).
//!
//! Every function that returns `i32` returns a `tfh_status`; on a non-zero status the calling thread's
//! `tfh_last_error` slot holds the payload of the matching `tenferro_device::Error` variant
//! (tenferro-device/src/lib.rs:108-159).
#![allow(non_camel_case_types)]

use std::os::raw::{c_char, c_void};

pub const TFH_MAX_RANK: usize = 16;

// ---- tfh_status: one per variant of tenferro_device::Error (tenferro-device/src/lib.rs:108-159)
pub const TFH_OK: i32 = 0;
pub const TFH_ERR_SHAPE_MISMATCH: i32 = 1;
pub const TFH_ERR_RANK_MISMATCH: i32 = 2;
pub const TFH_ERR_DEVICE: i32 = 3;
pub const TFH_ERR_NO_COMPATIBLE_DEVICE: i32 = 4;
pub const TFH_ERR_CROSS_MEMORY_SPACE: i32 = 5;
pub const TFH_ERR_INVALID_ARGUMENT: i32 = 6;
pub const TFH_ERR_STRIDED: i32 = 7;

// ---- tfh_dtype: the Standard-algebra scalar set (tenferro-algebra/src/lib.rs:58-72)
pub const TFH_F32: i32 = 0;
pub const TFH_F64: i32 = 1;
pub const TFH_C64: i32 = 2;
pub const TFH_C128: i32 = 3;

// ---- tfh_op: PrimDescriptor variants (tenferro-prims/src/lib.rs:152-245)
pub const TFH_OP_BATCHED_GEMM: i32 = 0;
pub const TFH_OP_REDUCE: i32 = 1;
pub const TFH_OP_TRACE: i32 = 2;
pub const TFH_OP_PERMUTE: i32 = 3;
pub const TFH_OP_ANTI_TRACE: i32 = 4;
pub const TFH_OP_ANTI_DIAG: i32 = 5;
pub const TFH_OP_CONTRACT: i32 = 6;
pub const TFH_OP_ELEMENTWISE_MUL: i32 = 7;

// ---- tfh_reduce_op, tfh_extension (tenferro-prims/src/lib.rs:100-128)
pub const TFH_REDUCE_SUM: i32 = 0;
pub const TFH_REDUCE_MAX: i32 = 1;
pub const TFH_REDUCE_MIN: i32 = 2;
pub const TFH_EXT_CONTRACT: i32 = 0;
pub const TFH_EXT_ELEMENTWISE_MUL: i32 = 1;

// ---- tfh_op_kind, tfh_space_kind, tfh_device_kind (tenferro-device/src/lib.rs:30-90)
pub const TFH_KIND_CONTRACT: i32 = 0;
pub const TFH_KIND_BATCHED_GEMM: i32 = 1;
pub const TFH_KIND_REDUCE: i32 = 2;
pub const TFH_KIND_TRACE: i32 = 3;
pub const TFH_KIND_PERMUTE: i32 = 4;
pub const TFH_KIND_ELEMENTWISE_MUL: i32 = 5;
pub const TFH_SPACE_MAIN_MEMORY: i32 = 0;
pub const TFH_SPACE_GPU_MEMORY: i32 = 1;
pub const TFH_DEVICE_CPU: i32 = 0;
pub const TFH_DEVICE_CUDA: i32 = 1;
pub const TFH_DEVICE_HIP: i32 = 2;

/// `tfh_view.flags`: read the (complex) input as its conjugate, without a conjugated copy.
pub const TFH_VIEW_CONJ: i32 = 1;
/// Size of the fixed device array `tfh_execute_static` takes its scratch from.
pub const TFH_STATIC_SCRATCH_BYTES: usize = 64 << 20;

/// Payload of the last failure on the calling thread.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct tfh_error_info {
    pub status: i32,
    pub n_expected: i32,
    pub n_got: i32,
    pub reserved: i32,
    pub expected: [i64; TFH_MAX_RANK],
    pub got: [i64; TFH_MAX_RANK],
    pub message: [c_char; 512],
}

/// The StridedView / StridedViewMut contract over a DEVICE base pointer (tenferro-tensor/src/lib.rs:169-171, 219-221):
/// element (i0, i1, ...) lives at `base + (offset + sum_d i_d * strides[d]) * size_of::<T>()`.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct tfh_view {
    pub base: *mut c_void,
    pub rank: i32,
    pub flags: i32,
    pub offset: i64,
    pub dims: [i64; TFH_MAX_RANK],
    pub strides: [i64; TFH_MAX_RANK],
}

/// PrimDescriptor flattened (tenferro-prims/src/lib.rs:152-245).  Permute's `modes_b` travels in `modes_c`.
#[repr(C)]
#[derive(Clone, Copy)]
pub struct tfh_desc {
    pub op: i32,
    pub reduce_op: i32,
    pub batch_dims: *const i64,
    pub n_batch_dims: i32,
    pub reserved: i32,
    pub m: i64,
    pub n: i64,
    pub k: i64,
    pub modes_a: *const u32,
    pub n_modes_a: i32,
    pub modes_b: *const u32,
    pub n_modes_b: i32,
    pub modes_c: *const u32,
    pub n_modes_c: i32,
    pub paired: *const u32,
    pub n_pairs: i32,
}

/// ComputeDevice as (tfh_device_kind, index) (tenferro-device/src/lib.rs:46-62).
#[repr(C)]
#[derive(Clone, Copy)]
pub struct tfh_compute_device {
    pub kind: i32,
    pub device_id: i32,
}

/// Opaque handles: created and destroyed by the library only.
#[repr(C)]
pub struct tfh_plan {
    _private: [u8; 0],
}
#[repr(C)]
pub struct tfh_subscripts {
    _private: [u8; 0],
}
#[repr(C)]
pub struct tfh_tree {
    _private: [u8; 0],
}
/// `hipStream_t`; null = the null stream.
pub type tfh_stream = *mut c_void;
/// `hipEvent_t`.
pub type tfh_event = *mut c_void;

extern "C" {
    // ---- errors, version, scalar types
    pub fn tfh_last_error(out: *mut tfh_error_info);
    pub fn tfh_status_name(status: i32) -> *const c_char;
    pub fn tfh_version() -> *const c_char;
    pub fn tfh_dtype_size(dtype: i32) -> usize;

    // ---- TensorPrims<Standard> for the Hip backend (tenferro-prims/src/lib.rs:278-340)
    pub fn tfh_has_extension(dtype: i32, ext: i32) -> i32;
    pub fn tfh_plan_create(dtype: i32, desc: *const tfh_desc, shapes: *const *const i64, ranks: *const i32,
        n_tensors: i32, out: *mut *mut tfh_plan) -> i32;
    pub fn tfh_plan_destroy(plan: *mut tfh_plan);
    pub fn tfh_plan_describe(plan: *const tfh_plan, buf: *mut c_char, cap: usize) -> i32;
    pub fn tfh_plan_cache_stats(plan: *const tfh_plan, hits: *mut i64, misses: *mut i64, entries: *mut i32) -> i32;
    pub fn tfh_execute(plan: *const tfh_plan, alpha: *const c_void, inputs: *const tfh_view, n_inputs: i32,
        beta: *const c_void, output: *mut tfh_view, stream: tfh_stream) -> i32;
    pub fn tfh_plan_create_grouped(dtype: i32, desc: *const tfh_desc, n_groups: i32, shapes: *const *const i64,
        ranks: *const i32, n_tensors: i32, out: *mut *mut tfh_plan) -> i32;
    pub fn tfh_execute_grouped(plan: *const tfh_plan, alpha: *const c_void, inputs: *const tfh_view, n_inputs: i32,
        beta: *const c_void, outputs: *mut tfh_view, stream: tfh_stream) -> i32;
    pub fn tfh_static_scratch_bytes() -> usize;
    pub fn tfh_execute_static(plan: *const tfh_plan, alpha: *const c_void, inputs: *const tfh_view, n_inputs: i32,
        beta: *const c_void, output: *mut tfh_view, stream: tfh_stream) -> i32;

    // ---- Tensor::conj / zeros / ones on device memory (tenferro-tensor/src/lib.rs:336-347, 622-658)
    pub fn tfh_conj(dtype: i32, input: *const tfh_view, out: *mut tfh_view, stream: tfh_stream) -> i32;
    pub fn tfh_fill(dtype: i32, value: *const c_void, out: *mut tfh_view, stream: tfh_stream) -> i32;

    // ---- Subscripts and ContractionTree (tenferro-einsum/src/lib.rs:239-356)
    pub fn tfh_subscripts_new(labels: *const u32, ranks: *const i32, n_inputs: i32, output: *const u32,
        n_output: i32, out: *mut *mut tfh_subscripts) -> i32;
    pub fn tfh_subscripts_parse(notation: *const c_char, out: *mut *mut tfh_subscripts) -> i32;
    pub fn tfh_subscripts_destroy(s: *mut tfh_subscripts);
    pub fn tfh_subscripts_n_inputs(s: *const tfh_subscripts) -> i32;
    pub fn tfh_subscripts_input_rank(s: *const tfh_subscripts, i: i32) -> i32;
    pub fn tfh_subscripts_labels(s: *const tfh_subscripts, i: i32, out: *mut u32, cap: i32) -> i32;
    pub fn tfh_subscripts_nesting(s: *const tfh_subscripts, buf: *mut c_char, cap: usize) -> i32;
    pub fn tfh_tree_optimize(s: *const tfh_subscripts, shapes: *const *const i64, ranks: *const i32, n_inputs: i32,
        out: *mut *mut tfh_tree) -> i32;
    pub fn tfh_tree_from_pairs(s: *const tfh_subscripts, shapes: *const *const i64, ranks: *const i32,
        n_inputs: i32, pairs: *const i32, n_pairs: i32, out: *mut *mut tfh_tree) -> i32;
    pub fn tfh_tree_destroy(t: *mut tfh_tree);
    pub fn tfh_tree_optimize_cached(s: *const tfh_subscripts, shapes: *const *const i64, ranks: *const i32,
        n_inputs: i32, out: *mut *mut tfh_tree) -> i32;
    pub fn tfh_tree_cache_stats(hits: *mut i64, misses: *mut i64, entries: *mut i64) -> i32;
    pub fn tfh_tree_cache_clear() -> i32;
    pub fn tfh_tree_n_inputs(t: *const tfh_tree) -> i32;
    pub fn tfh_tree_n_steps(t: *const tfh_tree) -> i32;
    pub fn tfh_tree_step(t: *const tfh_tree, i: i32, lhs: *mut i32, rhs: *mut i32) -> i32;
    pub fn tfh_tree_node(t: *const tfh_tree, node: i32, labels: *mut u32, dims: *mut i64, cap: i32) -> i32;
    pub fn tfh_tree_output_rank(t: *const tfh_tree) -> i32;
    pub fn tfh_tree_output_dims(t: *const tfh_tree, dims: *mut i64, cap: i32) -> i32;
    pub fn tfh_tree_mac_count(t: *const tfh_tree) -> f64;
    pub fn tfh_tree_peak_intermediate(t: *const tfh_tree) -> f64;

    // ---- the einsum executor (tenferro-einsum/src/lib.rs:393-621)
    pub fn tfh_einsum_execute(dtype: i32, tree: *const tfh_tree, operands: *const tfh_view, n_operands: i32,
        alpha: *const c_void, beta: *const c_void, output: *mut tfh_view, donate_mask: u64, stream: tfh_stream) -> i32;

    // ---- device model (tenferro-device/src/lib.rs:30-105)
    pub fn tfh_preferred_compute_devices(space_kind: i32, space_id: i64, op_kind: i32,
        out: *mut tfh_compute_device, cap: i32, n: *mut i32) -> i32;
    pub fn tfh_compute_device_format(kind: i32, device_id: i64, buf: *mut c_char, cap: usize) -> i32;
    pub fn tfh_device_count(n: *mut i32) -> i32;
    pub fn tfh_set_device(device_id: i32) -> i32;

    // ---- DataBuffer::Hip storage and transfers (tenferro-tensor/src/lib.rs:133-137, 660-671)
    pub fn tfh_malloc(bytes: usize, out: *mut *mut c_void) -> i32;
    pub fn tfh_free(ptr: *mut c_void) -> i32;
    pub fn tfh_memcpy_h2d(dst: *mut c_void, src: *const c_void, bytes: usize, stream: tfh_stream) -> i32;
    pub fn tfh_memcpy_d2h(dst: *mut c_void, src: *const c_void, bytes: usize, stream: tfh_stream) -> i32;
    pub fn tfh_memcpy_d2d(dst: *mut c_void, src: *const c_void, bytes: usize, stream: tfh_stream) -> i32;
    pub fn tfh_host_malloc(bytes: usize, out: *mut *mut c_void) -> i32;
    pub fn tfh_host_free(ptr: *mut c_void) -> i32;

    // ---- streams and CompletionEvent (tenferro-tensor/src/lib.rs:301-309, 677-713)
    pub fn tfh_stream_create(out: *mut tfh_stream) -> i32;
    pub fn tfh_stream_destroy(s: tfh_stream) -> i32;
    pub fn tfh_stream_synchronize(s: tfh_stream) -> i32;
    pub fn tfh_event_create(out: *mut tfh_event) -> i32;
    pub fn tfh_event_destroy(e: tfh_event) -> i32;
    pub fn tfh_event_record(e: tfh_event, s: tfh_stream) -> i32;
    pub fn tfh_event_synchronize(e: tfh_event) -> i32;
    pub fn tfh_event_query(e: tfh_event, ready: *mut i32) -> i32;
    pub fn tfh_stream_wait_event(s: tfh_stream, e: tfh_event) -> i32;

    // ---- measurement and diagnostics (no counterpart in the reference)
    pub fn tfh_profile_enable(on: i32) -> i32;
    pub fn tfh_profile_collect(kind: i32, total_ms: *mut f64, launches: *mut i32) -> i32;
    pub fn tfh_profile_kernel(kind: i32, index: i32, name: *mut c_char, cap: usize, total_ms: *mut f64,
        launches: *mut i32) -> i32;
    pub fn tfh_last_kernel() -> *const c_char;
    pub fn tfh_release_workspaces() -> i32;
}
