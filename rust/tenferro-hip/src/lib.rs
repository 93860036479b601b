//! AMD HIP (MI355X, gfx950) backend for the tenferro workspace.
//!
//! Safe wrappers over `tenferro-hip-sys` in the workspace's own vocabulary:
//!
//! - [`HipBackend`]: `impl TensorPrims<Standard>` (tenferro-prims/src/lib.rs:278-340), plus the two additions of the
//!   C library (grouped plans, the allocation-free execute).
//! - [`HipBuffer`]: the storage of `DataBuffer::Hip` (tenferro-tensor/src/lib.rs:133-137), with [`HipView`] /
//!   [`HipViewMut`] as the device-side `StridedView` / `StridedViewMut`.
//! - [`CompletionEvent`] and [`Stream`] (tenferro-tensor/src/lib.rs:301-309, 677-713).
//! - [`Subscripts`], [`ContractionTree`] and [`einsum_with_plan_into`] (tenferro-einsum/src/lib.rs:239-356, 584-621).
//! - [`preferred_compute_devices`] (tenferro-device/src/lib.rs:92-105) and [`check`], which turns a `tfh_status` into
//!   the matching `tenferro_device::Error` variant (tenferro-device/src/lib.rs:108-159).
//!
//! The crate is written against the reference workspace as it stands; it has not been compiled (the image the backend
//! is built in has no Rust toolchain).  `tests/test_rust_shim.py` of the backend's source tree checks the extern block
//! of `tenferro-hip-sys` against the C header symbol by symbol.

mod backend;
mod buffer;
mod einsum;
mod event;

pub use backend::{HipBackend, HipGroupedPlan, HipPlan};
pub use buffer::{HipBuffer, HipView, HipViewMut, PinnedBuffer};
pub use einsum::{einsum_with_plan_into, ContractionTree, Subscripts};
pub use event::{CompletionEvent, Stream};

use std::any::TypeId;
use std::ffi::CStr;
use std::mem::MaybeUninit;

use num_complex::{Complex32, Complex64};
use strided_view::StridedError;
use tenferro_device::{ComputeDevice, Error, LogicalMemorySpace, OpKind, Result};
use tenferro_hip_sys as sys;

/// The run-time tag a scalar type crosses the C boundary as (`tfh_dtype`): the Standard-algebra set
/// (tenferro-algebra/src/lib.rs:58-72).  The trait methods of `TensorPrims` are generic over every `ScalarBase`, so
/// the tag is looked up by `TypeId`; a type outside the set is an `InvalidArgument`, not a compile error.
pub fn dtype_tag<T: 'static>() -> Result<i32> {
    let t = TypeId::of::<T>();
    if t == TypeId::of::<f32>() {
        Ok(sys::TFH_F32)
    } else if t == TypeId::of::<f64>() {
        Ok(sys::TFH_F64)
    } else if t == TypeId::of::<Complex32>() {
        Ok(sys::TFH_C64)
    } else if t == TypeId::of::<Complex64>() {
        Ok(sys::TFH_C128)
    } else {
        Err(Error::InvalidArgument(format!(
            "the Hip backend computes on f32, f64, Complex32 and Complex64; got {}",
            std::any::type_name::<T>()
        )))
    }
}

fn space_from(kind: i64, id: i64) -> LogicalMemorySpace {
    if kind == sys::TFH_SPACE_GPU_MEMORY as i64 {
        LogicalMemorySpace::GpuMemory { space_id: id as usize }
    } else {
        LogicalMemorySpace::MainMemory
    }
}

fn space_parts(space: LogicalMemorySpace) -> (i32, i64) {
    match space {
        LogicalMemorySpace::MainMemory => (sys::TFH_SPACE_MAIN_MEMORY, 0),
        LogicalMemorySpace::GpuMemory { space_id } => (sys::TFH_SPACE_GPU_MEMORY, space_id as i64),
    }
}

fn op_kind_from(tag: i64) -> OpKind {
    match tag as i32 {
        sys::TFH_KIND_BATCHED_GEMM => OpKind::BatchedGemm,
        sys::TFH_KIND_REDUCE => OpKind::Reduce,
        sys::TFH_KIND_TRACE => OpKind::Trace,
        sys::TFH_KIND_PERMUTE => OpKind::Permute,
        sys::TFH_KIND_ELEMENTWISE_MUL => OpKind::ElementwiseMul,
        _ => OpKind::Contract,
    }
}

fn op_kind_tag(op: OpKind) -> i32 {
    match op {
        OpKind::Contract => sys::TFH_KIND_CONTRACT,
        OpKind::BatchedGemm => sys::TFH_KIND_BATCHED_GEMM,
        OpKind::Reduce => sys::TFH_KIND_REDUCE,
        OpKind::Trace => sys::TFH_KIND_TRACE,
        OpKind::Permute => sys::TFH_KIND_PERMUTE,
        OpKind::ElementwiseMul => sys::TFH_KIND_ELEMENTWISE_MUL,
    }
}

fn dims_of(v: &[i64; sys::TFH_MAX_RANK], n: i32) -> Vec<usize> {
    v[..(n.clamp(0, sys::TFH_MAX_RANK as i32) as usize)].iter().map(|&x| x as usize).collect()
}

fn message_of(info: &sys::tfh_error_info) -> String {
    // The library prefixes the text the way the Display impl of the variant does ("device error: ...",
    // "invalid argument: ..."); the variant's payload is the text without that prefix.
    let text = unsafe { CStr::from_ptr(info.message.as_ptr()) }.to_string_lossy().into_owned();
    for prefix in ["device error: ", "invalid argument: ", "strided: "] {
        if let Some(rest) = text.strip_prefix(prefix) {
            return rest.to_string();
        }
    }
    text
}

/// The two layout conditions the library reports with status 7: an output view with stride 0 on an axis longer than
/// one (its elements would alias), and a view whose base is not aligned to the element size.  Both are defects of the
/// (dims, strides, offset) triple, which is what `StridedError` describes; `strided-view` has no variant that carries
/// free text, so the closest structural variants are used and the library's own sentence stays available through
/// `tfh_last_error`.
fn strided_error(info: &sys::tfh_error_info) -> StridedError {
    let text = message_of(info);
    if text.contains("stride 0") {
        StridedError::StrideLengthMismatch
    } else {
        StridedError::OffsetOverflow
    }
}

/// `tfh_status` -> `tenferro_device::Error` (tenferro-device/src/lib.rs:108-159), one arm per variant.  The payload
/// comes from the calling thread's `tfh_last_error` slot, so this must run on the thread that made the failing call,
/// before any other call into the library.
pub fn check(status: i32) -> Result<()> {
    if status == sys::TFH_OK {
        return Ok(());
    }
    let mut slot = MaybeUninit::<sys::tfh_error_info>::zeroed();
    unsafe { sys::tfh_last_error(slot.as_mut_ptr()) };
    let info = unsafe { slot.assume_init() };
    Err(match status {
        sys::TFH_ERR_SHAPE_MISMATCH => Error::ShapeMismatch {
            expected: dims_of(&info.expected, info.n_expected),
            got: dims_of(&info.got, info.n_got),
        },
        sys::TFH_ERR_RANK_MISMATCH => Error::RankMismatch {
            expected: info.expected[0] as usize,
            got: info.got[0] as usize,
        },
        sys::TFH_ERR_DEVICE => Error::DeviceError(message_of(&info)),
        sys::TFH_ERR_NO_COMPATIBLE_DEVICE => Error::NoCompatibleComputeDevice {
            space: space_from(info.expected[0], info.expected[1]),
            op: op_kind_from(info.got[0]),
        },
        sys::TFH_ERR_CROSS_MEMORY_SPACE => Error::CrossMemorySpaceOperation {
            left: space_from(info.expected[0], info.expected[1]),
            right: space_from(info.got[0], info.got[1]),
        },
        sys::TFH_ERR_INVALID_ARGUMENT => Error::InvalidArgument(message_of(&info)),
        sys::TFH_ERR_STRIDED => Error::Strided(strided_error(&info)),
        other => Error::DeviceError(format!("unknown status {other}: {}", message_of(&info))),
    })
}

/// `preferred_compute_devices(space, op_kind)` (tenferro-device/src/lib.rs:92-105) as this backend answers it:
/// `GpuMemory { space_id: n }` -> `[Hip { device_id: n }]` when device n exists; `MainMemory` ->
/// `Error::NoCompatibleComputeDevice` (the library computes on HIP devices only -- the workspace-level function keeps
/// its CPU answer for main memory and asks here for GPU memory).
pub fn preferred_compute_devices(space: LogicalMemorySpace, op_kind: OpKind) -> Result<Vec<ComputeDevice>> {
    let (kind, id) = space_parts(space);
    let mut out = [sys::tfh_compute_device { kind: 0, device_id: 0 }; 8];
    let mut n = 0i32;
    check(unsafe {
        sys::tfh_preferred_compute_devices(kind, id, op_kind_tag(op_kind), out.as_mut_ptr(), out.len() as i32, &mut n)
    })?;
    Ok(out[..n as usize]
        .iter()
        .map(|d| match d.kind {
            sys::TFH_DEVICE_CPU => ComputeDevice::Cpu { device_id: d.device_id as usize },
            sys::TFH_DEVICE_CUDA => ComputeDevice::Cuda { device_id: d.device_id as usize },
            _ => ComputeDevice::Hip { device_id: d.device_id as usize },
        })
        .collect())
}

/// `Display for ComputeDevice` through the library ("hip:0"), for parity checks of the two spellings.
pub fn compute_device_string(device: ComputeDevice) -> Result<String> {
    let (kind, id) = match device {
        ComputeDevice::Cpu { device_id } => (sys::TFH_DEVICE_CPU, device_id),
        ComputeDevice::Cuda { device_id } => (sys::TFH_DEVICE_CUDA, device_id),
        ComputeDevice::Hip { device_id } => (sys::TFH_DEVICE_HIP, device_id),
    };
    let mut buf = [0 as std::os::raw::c_char; 32];
    check(unsafe { sys::tfh_compute_device_format(kind, id as i64, buf.as_mut_ptr(), buf.len()) })?;
    Ok(unsafe { CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned())
}

/// Number of HIP devices visible to the process.
pub fn device_count() -> Result<usize> {
    let mut n = 0i32;
    check(unsafe { sys::tfh_device_count(&mut n) })?;
    Ok(n as usize)
}

/// Makes `device_id` the calling thread's current device (allocations and launches go there).
pub fn set_device(device_id: usize) -> Result<()> {
    check(unsafe { sys::tfh_set_device(device_id as i32) })
}

/// "tenferro-hip 0.1 (gfx950)".
pub fn version() -> String {
    unsafe { CStr::from_ptr(sys::tfh_version()) }.to_string_lossy().into_owned()
}

/// Name of a status as the library spells it ("ShapeMismatch", ...).
pub fn status_name(status: i32) -> String {
    unsafe { CStr::from_ptr(sys::tfh_status_name(status)) }.to_string_lossy().into_owned()
}

/// Size in bytes of one element of a dtype tag.
pub fn dtype_size(tag: i32) -> usize {
    unsafe { sys::tfh_dtype_size(tag) }
}

/// Label of the dominant kernel most recently launched by the calling thread, e.g.
/// "(gemm128_kernel<double, true, false, true, 1, 1, 128>)".
pub fn last_kernel() -> String {
    unsafe { CStr::from_ptr(sys::tfh_last_kernel()) }.to_string_lossy().into_owned()
}

/// Frees the cached workspaces, intermediates and offset tables of every stream (buffers that belong to a captured
/// HIP graph are passed over).
pub fn release_workspaces() -> Result<()> {
    check(unsafe { sys::tfh_release_workspaces() })
}

/// Per-kernel timing of the library's own launches, for benchmarks.
pub mod profile {
    use super::{check, sys, Result};
    use std::ffi::CStr;

    /// Kinds of records: the dominant kernel of a contraction, of a copy/permute, of a reduction.
    #[derive(Debug, Clone, Copy, PartialEq, Eq)]
    pub enum Kind {
        Contract = 0,
        Copy = 1,
        Reduce = 2,
    }

    pub fn enable(on: bool) -> Result<()> {
        check(unsafe { sys::tfh_profile_enable(on as i32) })
    }

    /// The records of one kind by kernel, in order of first launch: (label, summed milliseconds, launches).
    /// Call before [`collect`], which forgets them.
    pub fn kernels(kind: Kind) -> Result<Vec<(String, f64, usize)>> {
        let mut out = Vec::new();
        for index in 0.. {
            let mut name = [0 as std::os::raw::c_char; 256];
            let (mut ms, mut launches) = (0f64, 0i32);
            check(unsafe {
                sys::tfh_profile_kernel(kind as i32, index, name.as_mut_ptr(), name.len(), &mut ms, &mut launches)
            })?;
            if launches == 0 {
                break;
            }
            out.push((unsafe { CStr::from_ptr(name.as_ptr()) }.to_string_lossy().into_owned(), ms, launches as usize));
        }
        Ok(out)
    }

    /// Summed duration and launch count of one kind since the last enable; waits for the launches and forgets them.
    pub fn collect(kind: Kind) -> Result<(f64, usize)> {
        let (mut ms, mut launches) = (0f64, 0i32);
        check(unsafe { sys::tfh_profile_collect(kind as i32, &mut ms, &mut launches) })?;
        Ok((ms, launches as usize))
    }
}
