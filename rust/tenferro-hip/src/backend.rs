//! `impl TensorPrims<Standard> for HipBackend` (tenferro-prims/src/lib.rs:278-340): describe -> plan -> execute on
//! one MI355X, with `output = alpha * op(inputs) + beta * output`.

use std::cell::Cell;
use std::ffi::{c_void, CStr};
use std::marker::PhantomData;

use strided_traits::ScalarBase;
use strided_view::{StridedView, StridedViewMut};
use tenferro_algebra::Standard;
use tenferro_device::{Error, Result};
use tenferro_hip_sys as sys;
use tenferro_prims::{Extension, PrimDescriptor, ReduceOp, TensorPrims};

use crate::buffer::{HipView, HipViewMut};
use crate::event::Stream;
use crate::{check, dtype_tag};

thread_local! {
    // The stream the trait methods enqueue on: `TensorPrims::execute` has no stream parameter.
    static CURRENT_STREAM: Cell<sys::tfh_stream> = const { Cell::new(std::ptr::null_mut()) };
}

/// The HIP backend.  All functions are associated functions, as for `CpuBackend` (tenferro-prims/src/lib.rs:413).
pub struct HipBackend;

/// Plan of the HIP backend: an immutable, thread-shareable handle; the kernel choice it stands for is made from the
/// descriptor and the shapes at `plan` time and from the views' strides at `execute` time.
pub struct HipPlan<T> {
    raw: *mut sys::tfh_plan,
    _scalar: PhantomData<T>,
}

unsafe impl<T> Send for HipPlan<T> {}
unsafe impl<T> Sync for HipPlan<T> {}

impl<T> HipPlan<T> {
    /// One line on what the plan launches (kernel family, GEMM view M/N/K/batch).
    pub fn describe(&self) -> String {
        let mut buf = [0 as std::os::raw::c_char; 256];
        unsafe { sys::tfh_plan_describe(self.raw, buf.as_mut_ptr(), buf.len()) };
        unsafe { CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }
    /// (executes that found their routed launch in the plan, executes that had to route, routes kept): the plan keeps
    /// the kernel selection of the first execute with each set of view strides (tenferro-prims/src/lib.rs:8, :284).
    pub fn cache_stats(&self) -> (i64, i64, i32) {
        let (mut h, mut m, mut e) = (0i64, 0i64, 0i32);
        unsafe { sys::tfh_plan_cache_stats(self.raw, &mut h, &mut m, &mut e) };
        (h, m, e)
    }
    pub(crate) fn raw(&self) -> *const sys::tfh_plan {
        self.raw
    }
}

impl<T> Drop for HipPlan<T> {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { sys::tfh_plan_destroy(self.raw) };
        }
    }
}

/// Plan over `n_groups` independent problems that share a descriptor but not their extents (the blocks of a
/// block-sparse contraction), executed in one launch.  No counterpart in `TensorPrims`.
pub struct HipGroupedPlan<T> {
    plan: HipPlan<T>,
    n_groups: usize,
    n_inputs: usize,
}

/// Keeps the arrays a `tfh_desc` points into alive for the duration of `tfh_plan_create`.
struct DescHolder {
    batch_dims: Vec<i64>,
    pairs: Vec<u32>,
    desc: sys::tfh_desc,
}

fn flatten(paired: &[(u32, u32)]) -> Vec<u32> {
    paired.iter().flat_map(|&(i, j)| [i, j]).collect()
}

impl DescHolder {
    /// `PrimDescriptor` (tenferro-prims/src/lib.rs:152-245) -> `tfh_desc`.  `Permute { modes_b }` travels in `modes_c`
    /// (the output's modes), as the header says.
    fn new(d: &PrimDescriptor) -> Box<Self> {
        let empty = sys::tfh_desc {
            op: 0,
            reduce_op: 0,
            batch_dims: std::ptr::null(),
            n_batch_dims: 0,
            reserved: 0,
            m: 0,
            n: 0,
            k: 0,
            modes_a: std::ptr::null(),
            n_modes_a: 0,
            modes_b: std::ptr::null(),
            n_modes_b: 0,
            modes_c: std::ptr::null(),
            n_modes_c: 0,
            paired: std::ptr::null(),
            n_pairs: 0,
        };
        // Boxed so that the pointers into `batch_dims` / `pairs` stay valid when the holder moves.
        let mut h = Box::new(Self { batch_dims: Vec::new(), pairs: Vec::new(), desc: empty });
        let set_modes = |desc: &mut sys::tfh_desc, a: &[u32], b: Option<&[u32]>, c: &[u32]| {
            desc.modes_a = a.as_ptr();
            desc.n_modes_a = a.len() as i32;
            if let Some(b) = b {
                desc.modes_b = b.as_ptr();
                desc.n_modes_b = b.len() as i32;
            }
            desc.modes_c = c.as_ptr();
            desc.n_modes_c = c.len() as i32;
        };
        match d {
            PrimDescriptor::BatchedGemm { batch_dims, m, n, k } => {
                h.batch_dims = batch_dims.iter().map(|&x| x as i64).collect();
                h.desc.op = sys::TFH_OP_BATCHED_GEMM;
                h.desc.batch_dims = h.batch_dims.as_ptr();
                h.desc.n_batch_dims = h.batch_dims.len() as i32;
                h.desc.m = *m as i64;
                h.desc.n = *n as i64;
                h.desc.k = *k as i64;
            }
            PrimDescriptor::Reduce { modes_a, modes_c, op } => {
                h.desc.op = sys::TFH_OP_REDUCE;
                h.desc.reduce_op = match op {
                    ReduceOp::Sum => sys::TFH_REDUCE_SUM,
                    ReduceOp::Max => sys::TFH_REDUCE_MAX,
                    ReduceOp::Min => sys::TFH_REDUCE_MIN,
                };
                set_modes(&mut h.desc, modes_a, None, modes_c);
            }
            PrimDescriptor::Trace { modes_a, modes_c, paired }
            | PrimDescriptor::AntiTrace { modes_a, modes_c, paired }
            | PrimDescriptor::AntiDiag { modes_a, modes_c, paired } => {
                h.desc.op = match d {
                    PrimDescriptor::Trace { .. } => sys::TFH_OP_TRACE,
                    PrimDescriptor::AntiTrace { .. } => sys::TFH_OP_ANTI_TRACE,
                    _ => sys::TFH_OP_ANTI_DIAG,
                };
                h.pairs = flatten(paired);
                h.desc.paired = h.pairs.as_ptr();
                h.desc.n_pairs = paired.len() as i32;
                set_modes(&mut h.desc, modes_a, None, modes_c);
            }
            PrimDescriptor::Permute { modes_a, modes_b } => {
                h.desc.op = sys::TFH_OP_PERMUTE;
                set_modes(&mut h.desc, modes_a, None, modes_b);
            }
            PrimDescriptor::Contract { modes_a, modes_b, modes_c } => {
                h.desc.op = sys::TFH_OP_CONTRACT;
                set_modes(&mut h.desc, modes_a, Some(modes_b), modes_c);
            }
            PrimDescriptor::ElementwiseMul => {
                h.desc.op = sys::TFH_OP_ELEMENTWISE_MUL;
            }
        }
        h
    }
}

/// Shapes as the C side takes them: one pointer and one rank per tensor, extents as i64.
struct Shapes {
    _dims: Vec<Vec<i64>>,
    ptrs: Vec<*const i64>,
    ranks: Vec<i32>,
}

impl Shapes {
    fn new<'s>(shapes: impl Iterator<Item = &'s [usize]>) -> Self {
        let dims: Vec<Vec<i64>> = shapes.map(|s| s.iter().map(|&x| x as i64).collect()).collect();
        let ptrs = dims.iter().map(|d| d.as_ptr()).collect();
        let ranks = dims.iter().map(|d| d.len() as i32).collect();
        Self { _dims: dims, ptrs, ranks }
    }
}

impl TensorPrims<Standard> for HipBackend {
    type Plan<T: ScalarBase> = HipPlan<T>;

    /// tenferro-prims/src/lib.rs:282-298.  Validates the descriptor against the shapes (inputs first, then the
    /// output); touches no device.
    fn plan<T: ScalarBase>(desc: &PrimDescriptor, shapes: &[&[usize]]) -> Result<HipPlan<T>> {
        let tag = dtype_tag::<T>()?;
        let holder = DescHolder::new(desc);
        let s = Shapes::new(shapes.iter().copied());
        let mut raw: *mut sys::tfh_plan = std::ptr::null_mut();
        check(unsafe {
            sys::tfh_plan_create(tag, &holder.desc, s.ptrs.as_ptr(), s.ranks.as_ptr(), shapes.len() as i32, &mut raw)
        })?;
        Ok(HipPlan { raw, _scalar: PhantomData })
    }

    /// tenferro-prims/src/lib.rs:300-320.  The views look into DEVICE memory (`HipBuffer::as_device_slice`); the
    /// kernels are enqueued on the calling thread's current stream ([`HipBackend::set_current_stream`]) and the call
    /// does not wait for them.
    ///
    /// # Device memory
    /// The trait's signature cannot say where a `StridedView` lives.  This backend takes the ADDRESSES of the views'
    /// slices as device addresses: every view handed to it must have been built over
    /// [`HipBuffer::as_device_slice`] / [`HipBuffer::as_device_slice_mut`] (both `unsafe`, which is where the caller
    /// takes on that obligation).  A view over ordinary host memory makes the kernels dereference host pointers.  The
    /// tensor and einsum layers never go through this method: they call [`HipBackend::execute_on`] with [`HipView`]s,
    /// which can only be made from a `HipBuffer`.
    fn execute<T: ScalarBase>(
        plan: &HipPlan<T>,
        alpha: T,
        inputs: &[&StridedView<T>],
        beta: T,
        output: &mut StridedViewMut<T>,
    ) -> Result<()> {
        let views = inputs.iter().map(|v| HipView::from_strided(v)).collect::<Result<Vec<_>>>()?;
        let refs: Vec<&HipView<T>> = views.iter().collect();
        let mut out = HipViewMut::from_strided(output)?;
        let stream = unsafe { Stream::from_raw(CURRENT_STREAM.with(|c| c.get())) };
        Self::execute_on(plan, alpha, &refs, beta, &mut out, &stream)
    }

    /// tenferro-prims/src/lib.rs:322-339: Contract and ElementwiseMul are available for the four Standard scalars.
    fn has_extension_for<T: ScalarBase>(ext: Extension) -> bool {
        let ext = match ext {
            Extension::Contract => sys::TFH_EXT_CONTRACT,
            Extension::ElementwiseMul => sys::TFH_EXT_ELEMENTWISE_MUL,
        };
        match dtype_tag::<T>() {
            Ok(tag) => unsafe { sys::tfh_has_extension(tag, ext) != 0 },
            Err(_) => false,
        }
    }
}

impl HipBackend {
    /// The stream `TensorPrims::execute` enqueues on from the calling thread (the null stream until set).  The stream
    /// must outlive its use here.
    pub fn set_current_stream(stream: &Stream) {
        CURRENT_STREAM.with(|c| c.set(stream.raw()));
    }

    /// `execute` on device views and an explicit stream: what the trait method forwards to, and what the tensor and
    /// einsum layers call directly (a `Tensor` with `DataBuffer::Hip` hands out `HipView`s, which also carry the
    /// conjugate-on-load flag that `StridedView` has no room for).
    pub fn execute_on<T: ScalarBase>(
        plan: &HipPlan<T>,
        alpha: T,
        inputs: &[&HipView<T>],
        beta: T,
        output: &mut HipViewMut<T>,
        stream: &Stream,
    ) -> Result<()> {
        let raw_inputs: Vec<sys::tfh_view> = inputs.iter().map(|v| v.raw()).collect();
        let mut raw_output = output.raw();
        check(unsafe {
            sys::tfh_execute(
                plan.raw(),
                &alpha as *const T as *const c_void,
                raw_inputs.as_ptr(),
                raw_inputs.len() as i32,
                &beta as *const T as *const c_void,
                &mut raw_output,
                stream.raw(),
            )
        })
    }

    /// `execute_on` for callers that cannot allocate device memory (under HIP graph capture, in serving loops): the
    /// call's scratch comes from one fixed array of [`HipBackend::static_scratch_bytes`] per device.  A call that
    /// needs more is an `InvalidArgument`; calls that overlap in time on one device race on the array.
    pub fn execute_static<T: ScalarBase>(
        plan: &HipPlan<T>,
        alpha: T,
        inputs: &[&HipView<T>],
        beta: T,
        output: &mut HipViewMut<T>,
        stream: &Stream,
    ) -> Result<()> {
        let raw_inputs: Vec<sys::tfh_view> = inputs.iter().map(|v| v.raw()).collect();
        let mut raw_output = output.raw();
        check(unsafe {
            sys::tfh_execute_static(
                plan.raw(),
                &alpha as *const T as *const c_void,
                raw_inputs.as_ptr(),
                raw_inputs.len() as i32,
                &beta as *const T as *const c_void,
                &mut raw_output,
                stream.raw(),
            )
        })
    }

    pub fn static_scratch_bytes() -> usize {
        unsafe { sys::tfh_static_scratch_bytes() }
    }

    /// Grouped plan: `group_shapes[g]` holds the shapes of group g's tensors, inputs first, then the output.
    pub fn plan_grouped<T: ScalarBase>(desc: &PrimDescriptor, group_shapes: &[&[&[usize]]]) -> Result<HipGroupedPlan<T>> {
        let tag = dtype_tag::<T>()?;
        let n_tensors = group_shapes.first().map_or(0, |g| g.len());
        if group_shapes.iter().any(|g| g.len() != n_tensors) {
            return Err(Error::InvalidArgument("every group of a grouped plan has the same number of tensors".into()));
        }
        let holder = DescHolder::new(desc);
        let s = Shapes::new(group_shapes.iter().flat_map(|g| g.iter().copied()));
        let mut raw: *mut sys::tfh_plan = std::ptr::null_mut();
        check(unsafe {
            sys::tfh_plan_create_grouped(
                tag,
                &holder.desc,
                group_shapes.len() as i32,
                s.ptrs.as_ptr(),
                s.ranks.as_ptr(),
                n_tensors as i32,
                &mut raw,
            )
        })?;
        Ok(HipGroupedPlan {
            plan: HipPlan { raw, _scalar: PhantomData },
            n_groups: group_shapes.len(),
            n_inputs: n_tensors.saturating_sub(1),
        })
    }

    /// One launch over all groups: `inputs[g]` are group g's input views, `outputs[g]` its output view.
    pub fn execute_grouped<T: ScalarBase>(
        plan: &HipGroupedPlan<T>,
        alpha: T,
        inputs: &[&[&HipView<T>]],
        beta: T,
        outputs: &mut [HipViewMut<T>],
        stream: &Stream,
    ) -> Result<()> {
        if inputs.len() != plan.n_groups || outputs.len() != plan.n_groups {
            return Err(Error::InvalidArgument(format!(
                "grouped plan over {} groups, got {} input groups and {} outputs",
                plan.n_groups,
                inputs.len(),
                outputs.len()
            )));
        }
        if inputs.iter().any(|g| g.len() != plan.n_inputs) {
            return Err(Error::InvalidArgument(format!("each group takes {} inputs", plan.n_inputs)));
        }
        let raw_inputs: Vec<sys::tfh_view> = inputs.iter().flat_map(|g| g.iter().map(|v| v.raw())).collect();
        let mut raw_outputs: Vec<sys::tfh_view> = outputs.iter().map(|v| v.raw()).collect();
        check(unsafe {
            sys::tfh_execute_grouped(
                plan.plan.raw(),
                &alpha as *const T as *const c_void,
                raw_inputs.as_ptr(),
                plan.n_inputs as i32,
                &beta as *const T as *const c_void,
                raw_outputs.as_mut_ptr(),
                stream.raw(),
            )
        })
    }
}
