//! The device side of `tenferro-einsum`: `Subscripts`, `ContractionTree` and the one executor call every `einsum*`
//! entry point ends in (tenferro-einsum/src/lib.rs:239-356, 393-621).  The nine public functions of that crate
//! differ in how they obtain the tree (string, subscripts, pre-built), who owns the operands (`_owned`: set the
//! operand's bit in `donate_mask`) and who allocates the output (`_into`: the caller); for `GpuMemory` operands each
//! reduces to [`einsum_with_plan_into`].

use std::ffi::{c_void, CStr, CString};

use strided_traits::ScalarBase;
use tenferro_device::{Error, Result};
use tenferro_hip_sys as sys;

use crate::buffer::{HipView, HipViewMut};
use crate::event::Stream;
use crate::{check, dtype_tag};

/// Parsed einsum subscripts held by the library (tenferro-einsum/src/lib.rs:239-283), including the parenthesised
/// pairwise order of notations like "ij,(jk,kl)->il".
pub struct Subscripts {
    raw: *mut sys::tfh_subscripts,
}

unsafe impl Send for Subscripts {}
unsafe impl Sync for Subscripts {}

impl Subscripts {
    /// `Subscripts::new(inputs, output)` (:253-258).
    pub fn new(inputs: &[&[u32]], output: &[u32]) -> Result<Self> {
        let labels: Vec<u32> = inputs.iter().flat_map(|s| s.iter().copied()).collect();
        let ranks: Vec<i32> = inputs.iter().map(|s| s.len() as i32).collect();
        let mut raw = std::ptr::null_mut();
        check(unsafe {
            sys::tfh_subscripts_new(labels.as_ptr(), ranks.as_ptr(), inputs.len() as i32, output.as_ptr(), output.len() as i32, &mut raw)
        })?;
        Ok(Self { raw })
    }

    /// `Subscripts::parse(notation)` (:260-283).  Malformed notation is an `InvalidArgument`.
    pub fn parse(notation: &str) -> Result<Self> {
        let text = CString::new(notation).map_err(|_| Error::InvalidArgument("notation contains a NUL byte".into()))?;
        let mut raw = std::ptr::null_mut();
        check(unsafe { sys::tfh_subscripts_parse(text.as_ptr(), &mut raw) })?;
        Ok(Self { raw })
    }

    pub fn n_inputs(&self) -> usize {
        unsafe { sys::tfh_subscripts_n_inputs(self.raw) as usize }
    }

    fn labels_of(&self, index: i32) -> Vec<u32> {
        let mut out = vec![0u32; sys::TFH_MAX_RANK];
        let rank = unsafe { sys::tfh_subscripts_labels(self.raw, index, out.as_mut_ptr(), out.len() as i32) };
        out.truncate(rank.max(0) as usize);
        out
    }

    /// The `inputs` field of the reference struct (:241).
    pub fn inputs(&self) -> Vec<Vec<u32>> {
        (0..self.n_inputs())
            .map(|i| {
                debug_assert_eq!(unsafe { sys::tfh_subscripts_input_rank(self.raw, i as i32) } as usize, self.labels_of(i as i32).len());
                self.labels_of(i as i32)
            })
            .collect()
    }

    /// The `output` field of the reference struct (:243).
    pub fn output(&self) -> Vec<u32> {
        self.labels_of(-1)
    }

    /// The parenthesisation as written, operands by index: "ij,(jk,kl)->il" gives "0,(1,2)".
    pub fn nesting(&self) -> String {
        let mut buf = [0 as std::os::raw::c_char; 512];
        unsafe { sys::tfh_subscripts_nesting(self.raw, buf.as_mut_ptr(), buf.len()) };
        unsafe { CStr::from_ptr(buf.as_ptr()) }.to_string_lossy().into_owned()
    }
}

impl Drop for Subscripts {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { sys::tfh_subscripts_destroy(self.raw) };
        }
    }
}

fn marshal(shapes: &[&[usize]]) -> (Vec<Vec<i64>>, Vec<i32>) {
    let dims: Vec<Vec<i64>> = shapes.iter().map(|s| s.iter().map(|&x| x as i64).collect()).collect();
    let ranks = dims.iter().map(|d| d.len() as i32).collect();
    (dims, ranks)
}

/// A pairwise contraction order (tenferro-einsum/src/lib.rs:297-356); immutable and reference counted inside the
/// library, so a tree from the cache stays valid for its holders.
pub struct ContractionTree {
    raw: *mut sys::tfh_tree,
}

unsafe impl Send for ContractionTree {}
unsafe impl Sync for ContractionTree {}

impl ContractionTree {
    /// `ContractionTree::optimize` (:303-318): minimum total operation count, exhaustive up to 12 operands.
    pub fn optimize(subscripts: &Subscripts, shapes: &[&[usize]]) -> Result<Self> {
        let (dims, ranks) = marshal(shapes);
        let ptrs: Vec<*const i64> = dims.iter().map(|d| d.as_ptr()).collect();
        let mut raw = std::ptr::null_mut();
        check(unsafe { sys::tfh_tree_optimize(subscripts.raw, ptrs.as_ptr(), ranks.as_ptr(), shapes.len() as i32, &mut raw) })?;
        Ok(Self { raw })
    }

    /// The same tree from the process-wide cache keyed on (labels, grouping, shapes): what `einsum` and
    /// `einsum_with_subscripts` use, since they would otherwise optimise the same network on every call.
    pub fn optimize_cached(subscripts: &Subscripts, shapes: &[&[usize]]) -> Result<Self> {
        let (dims, ranks) = marshal(shapes);
        let ptrs: Vec<*const i64> = dims.iter().map(|d| d.as_ptr()).collect();
        let mut raw = std::ptr::null_mut();
        check(unsafe {
            sys::tfh_tree_optimize_cached(subscripts.raw, ptrs.as_ptr(), ranks.as_ptr(), shapes.len() as i32, &mut raw)
        })?;
        Ok(Self { raw })
    }

    /// `ContractionTree::from_pairs` (:320-355): intermediates are numbered from `n_inputs` upward.
    pub fn from_pairs(subscripts: &Subscripts, shapes: &[&[usize]], pairs: &[(usize, usize)]) -> Result<Self> {
        let (dims, ranks) = marshal(shapes);
        let ptrs: Vec<*const i64> = dims.iter().map(|d| d.as_ptr()).collect();
        let flat: Vec<i32> = pairs.iter().flat_map(|&(l, r)| [l as i32, r as i32]).collect();
        let mut raw = std::ptr::null_mut();
        check(unsafe {
            sys::tfh_tree_from_pairs(
                subscripts.raw,
                ptrs.as_ptr(),
                ranks.as_ptr(),
                shapes.len() as i32,
                flat.as_ptr(),
                pairs.len() as i32,
                &mut raw,
            )
        })?;
        Ok(Self { raw })
    }

    pub fn n_inputs(&self) -> usize {
        unsafe { sys::tfh_tree_n_inputs(self.raw) as usize }
    }

    /// The steps in execution order: step i contracts operands (lhs, rhs) into intermediate `n_inputs + i`.
    pub fn steps(&self) -> Vec<(usize, usize)> {
        let n = unsafe { sys::tfh_tree_n_steps(self.raw) };
        (0..n)
            .map(|i| {
                let (mut l, mut r) = (0i32, 0i32);
                unsafe { sys::tfh_tree_step(self.raw, i, &mut l, &mut r) };
                (l as usize, r as usize)
            })
            .collect()
    }

    /// Labels and extents of a node (input, intermediate, or the result = the last node).
    pub fn node(&self, node: usize) -> (Vec<u32>, Vec<usize>) {
        let mut labels = vec![0u32; 64];
        let mut dims = vec![0i64; 64];
        let rank = unsafe { sys::tfh_tree_node(self.raw, node as i32, labels.as_mut_ptr(), dims.as_mut_ptr(), 64) }.max(0) as usize;
        labels.truncate(rank);
        (labels, dims[..rank].iter().map(|&d| d as usize).collect())
    }

    /// Shape of the result, in the requested output order: what the allocating `einsum*` forms size their output by.
    pub fn output_dims(&self) -> Vec<usize> {
        let rank = unsafe { sys::tfh_tree_output_rank(self.raw) }.max(0) as usize;
        let mut dims = vec![0i64; rank.max(1)];
        unsafe { sys::tfh_tree_output_dims(self.raw, dims.as_mut_ptr(), dims.len() as i32) };
        dims[..rank].iter().map(|&d| d as usize).collect()
    }

    /// Scalar multiply-adds of the whole tree (a complex one counts once).
    pub fn mac_count(&self) -> f64 {
        unsafe { sys::tfh_tree_mac_count(self.raw) }
    }

    /// Element count of the largest intermediate.
    pub fn peak_intermediate(&self) -> f64 {
        unsafe { sys::tfh_tree_peak_intermediate(self.raw) }
    }

    /// (hits, misses, entries) of the process-wide tree cache.
    pub fn cache_stats() -> Result<(i64, i64, i64)> {
        let (mut h, mut m, mut e) = (0i64, 0i64, 0i64);
        check(unsafe { sys::tfh_tree_cache_stats(&mut h, &mut m, &mut e) })?;
        Ok((h, m, e))
    }

    pub fn cache_clear() -> Result<()> {
        check(unsafe { sys::tfh_tree_cache_clear() })
    }
}

impl Drop for ContractionTree {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { sys::tfh_tree_destroy(self.raw) };
        }
    }
}

/// `einsum_with_plan_into` (tenferro-einsum/src/lib.rs:584-621) for operands in GPU memory:
/// `output = alpha * einsum(operands) + beta * output`.  Every pairwise step is enqueued on `stream`, intermediates
/// stay in device memory and the host never waits: the caller makes `stream` wait for the operands' pending
/// `CompletionEvent`s first ([`Stream::wait_event`]) and records a fresh one for the output afterwards.
///
/// `donate_mask`: bit i set = operand i's buffer may be overwritten with an intermediate (the `_owned` variants,
/// :436-498, when the operand is the sole owner of a dense buffer).
pub fn einsum_with_plan_into<T: ScalarBase>(
    tree: &ContractionTree,
    operands: &[&HipView<T>],
    alpha: T,
    beta: T,
    output: &mut HipViewMut<T>,
    donate_mask: u64,
    stream: &Stream,
) -> Result<()> {
    let views: Vec<sys::tfh_view> = operands.iter().map(|v| v.raw()).collect();
    let mut out = output.raw();
    check(unsafe {
        sys::tfh_einsum_execute(
            dtype_tag::<T>()?,
            tree.raw,
            views.as_ptr(),
            views.len() as i32,
            &alpha as *const T as *const c_void,
            &beta as *const T as *const c_void,
            &mut out,
            donate_mask,
            stream.raw(),
        )
    })
}
