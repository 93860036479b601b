//! Device storage: `HipBuffer<T>` is what the `Hip(HipBuffer<T>)` variant of `DataBuffer`
//! (tenferro-tensor/src/lib.rs:133-137, marked "future" there) holds, and `HipView` / `HipViewMut` are the
//! `StridedView` / `StridedViewMut` contract (dims as usize, strides and offset as isize in units of T,
//! tenferro-tensor/src/lib.rs:169-171, 219-221) over its device pointer.

use std::ffi::c_void;
use std::marker::PhantomData;

use strided_traits::ScalarBase;
use strided_view::{StridedView, StridedViewMut};
use tenferro_device::{Error, LogicalMemorySpace, Result};
use tenferro_hip_sys as sys;

use crate::event::Stream;
use crate::{check, dtype_tag};

/// An owned allocation of `len` elements of `T` in the memory of one HIP device.
///
/// The pointer is a device address: it is never dereferenced on the host.  Dropping the buffer frees it
/// (`tfh_free`), which waits for nothing: the owner (a `Tensor` with a pending `CompletionEvent`) waits for or
/// chains behind the kernels that still use it first, as `Tensor::wait` does (tenferro-tensor/src/lib.rs:677-704).
pub struct HipBuffer<T> {
    ptr: *mut T,
    len: usize,
    device_id: usize,
}

// The buffer is plain device memory; the library's entry points may be called from any thread.
unsafe impl<T: Send> Send for HipBuffer<T> {}
unsafe impl<T: Sync> Sync for HipBuffer<T> {}

impl<T: ScalarBase> HipBuffer<T> {
    /// Uninitialised device memory for `len` elements on the current device.
    pub fn new(len: usize, device_id: usize) -> Result<Self> {
        crate::set_device(device_id)?;
        let mut raw: *mut c_void = std::ptr::null_mut();
        check(unsafe { sys::tfh_malloc(len * std::mem::size_of::<T>(), &mut raw) })?;
        Ok(Self { ptr: raw as *mut T, len, device_id })
    }

    /// `Tensor::zeros` / `ones` (tenferro-tensor/src/lib.rs:336-347) on device memory: every element = `value`.
    pub fn filled(len: usize, value: T, device_id: usize, stream: &Stream) -> Result<Self> {
        let buf = Self::new(len, device_id)?;
        let mut v = HipViewMut::dense(&buf, &[len]).raw();
        check(unsafe { sys::tfh_fill(dtype_tag::<T>()?, &value as *const T as *const c_void, &mut v, stream.raw()) })?;
        Ok(buf)
    }

    /// Host -> device (`Tensor::to_memory_space_async`, tenferro-tensor/src/lib.rs:660-671).  Pageable host memory is
    /// staged through the stream's pinned buffers and the call returns when `data` may be reused; memory from
    /// [`PinnedBuffer`] is handed to the copy engine directly and the call returns at once.
    pub fn from_host(data: &[T], device_id: usize, stream: &Stream) -> Result<Self> {
        let buf = Self::new(data.len(), device_id)?;
        check(unsafe {
            sys::tfh_memcpy_h2d(buf.ptr as *mut c_void, data.as_ptr() as *const c_void, std::mem::size_of_val(data), stream.raw())
        })?;
        Ok(buf)
    }

    /// Device -> host into `out` (same length).  For pageable `out` the data is there on return; for pinned memory
    /// the transfer completes in stream order (record an event and wait for it).
    pub fn copy_to_host(&self, out: &mut [T], stream: &Stream) -> Result<()> {
        if out.len() != self.len {
            return Err(Error::ShapeMismatch { expected: vec![self.len], got: vec![out.len()] });
        }
        check(unsafe {
            sys::tfh_memcpy_d2h(out.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, self.len * std::mem::size_of::<T>(), stream.raw())
        })
    }

    /// A copy on the same device, in stream order.
    pub fn duplicate(&self, stream: &Stream) -> Result<Self> {
        let buf = Self::new(self.len, self.device_id)?;
        check(unsafe {
            sys::tfh_memcpy_d2d(buf.ptr as *mut c_void, self.ptr as *const c_void, self.len * std::mem::size_of::<T>(), stream.raw())
        })?;
        Ok(buf)
    }

    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn device_id(&self) -> usize {
        self.device_id
    }
    pub fn logical_memory_space(&self) -> LogicalMemorySpace {
        LogicalMemorySpace::GpuMemory { space_id: self.device_id }
    }
    pub fn as_device_ptr(&self) -> *mut T {
        self.ptr
    }

    /// The buffer as the `&[T]` a `StridedView` is built over, for passing device tensors through the signature of
    /// `TensorPrims::execute` (tenferro-prims/src/lib.rs:314-320).
    ///
    /// # Safety
    /// The slice covers DEVICE memory.  It may only be handed to `HipBackend`, which takes its address and never
    /// reads through it; reading or writing an element on the host is undefined behaviour.
    pub unsafe fn as_device_slice(&self) -> &[T] {
        std::slice::from_raw_parts(self.ptr, self.len)
    }

    /// Mutable counterpart of [`as_device_slice`](Self::as_device_slice); same contract.
    ///
    /// # Safety
    /// As for `as_device_slice`.
    pub unsafe fn as_device_slice_mut(&mut self) -> &mut [T] {
        std::slice::from_raw_parts_mut(self.ptr, self.len)
    }
}

impl<T> Drop for HipBuffer<T> {
    fn drop(&mut self) {
        if !self.ptr.is_null() {
            // A failure to free cannot be reported from drop; the library keeps it in tfh_last_error.
            unsafe { sys::tfh_free(self.ptr as *mut c_void) };
        }
    }
}

/// Page-locked host memory (`tfh_host_malloc`): transfers from and to it go to the copy engine directly and overlap
/// kernels of other streams.  A `MainMemory` tensor that is meant to move to the device may keep its data here.
pub struct PinnedBuffer<T> {
    ptr: *mut T,
    len: usize,
}

unsafe impl<T: Send> Send for PinnedBuffer<T> {}

impl<T: Copy> PinnedBuffer<T> {
    pub fn new(len: usize) -> Result<Self> {
        let mut raw: *mut c_void = std::ptr::null_mut();
        check(unsafe { sys::tfh_host_malloc(len * std::mem::size_of::<T>(), &mut raw) })?;
        unsafe { std::ptr::write_bytes(raw as *mut u8, 0, len * std::mem::size_of::<T>()) };
        Ok(Self { ptr: raw as *mut T, len })
    }
    pub fn as_slice(&self) -> &[T] {
        unsafe { std::slice::from_raw_parts(self.ptr, self.len) }
    }
    pub fn as_mut_slice(&mut self) -> &mut [T] {
        unsafe { std::slice::from_raw_parts_mut(self.ptr, self.len) }
    }
}

impl<T> Drop for PinnedBuffer<T> {
    fn drop(&mut self) {
        if !self.ptr.is_null() {
            unsafe { sys::tfh_host_free(self.ptr as *mut c_void) };
        }
    }
}

/// A read-only strided view of device memory, lifetime-tied to the buffer it looks into.
#[derive(Clone)]
pub struct HipView<'a, T> {
    base: *const T,
    dims: Vec<usize>,
    strides: Vec<isize>,
    offset: isize,
    conj: bool,
    _buffer: PhantomData<&'a HipBuffer<T>>,
}

/// A writable strided view of device memory.
pub struct HipViewMut<'a, T> {
    base: *mut T,
    dims: Vec<usize>,
    strides: Vec<isize>,
    offset: isize,
    _buffer: PhantomData<&'a mut HipBuffer<T>>,
}

fn row_major(dims: &[usize]) -> Vec<isize> {
    let mut strides = vec![1isize; dims.len()];
    for d in (0..dims.len().saturating_sub(1)).rev() {
        strides[d] = strides[d + 1] * dims[d + 1] as isize;
    }
    strides
}

fn fill_raw(base: *mut c_void, dims: &[usize], strides: &[isize], offset: isize, flags: i32) -> sys::tfh_view {
    let mut v = sys::tfh_view {
        base,
        rank: dims.len() as i32,
        flags,
        offset: offset as i64,
        dims: [0; sys::TFH_MAX_RANK],
        strides: [0; sys::TFH_MAX_RANK],
    };
    for (i, (&d, &s)) in dims.iter().zip(strides).enumerate().take(sys::TFH_MAX_RANK) {
        v.dims[i] = d as i64;
        v.strides[i] = s as i64;
    }
    v
}

fn check_rank(rank: usize) -> Result<()> {
    if rank > sys::TFH_MAX_RANK {
        return Err(Error::InvalidArgument(format!("rank {rank} is above the {} the Hip backend takes", sys::TFH_MAX_RANK)));
    }
    Ok(())
}

impl<'a, T: ScalarBase> HipView<'a, T> {
    pub fn new(buffer: &'a HipBuffer<T>, dims: &[usize], strides: &[isize], offset: isize) -> Result<Self> {
        check_rank(dims.len())?;
        if dims.len() != strides.len() {
            return Err(Error::RankMismatch { expected: dims.len(), got: strides.len() });
        }
        Ok(Self { base: buffer.as_device_ptr(), dims: dims.to_vec(), strides: strides.to_vec(), offset, conj: false, _buffer: PhantomData })
    }

    /// The whole buffer as a dense row-major tensor of shape `dims`.
    pub fn dense(buffer: &'a HipBuffer<T>, dims: &[usize]) -> Self {
        Self { base: buffer.as_device_ptr(), dims: dims.to_vec(), strides: row_major(dims), offset: 0, conj: false, _buffer: PhantomData }
    }

    /// From the `StridedView` that `TensorPrims::execute` is handed: the slice under it is device memory
    /// ([`HipBuffer::as_device_slice`]); only its address, dims, strides and offset are read.
    pub fn from_strided<'v>(view: &'a StridedView<'v, T>) -> Result<Self>
    where
        'v: 'a,
    {
        check_rank(view.dims().len())?;
        Ok(Self {
            base: view.data().as_ptr(),
            dims: view.dims().to_vec(),
            strides: view.strides().to_vec(),
            offset: view.offset(),
            conj: false,
            _buffer: PhantomData,
        })
    }

    /// The same elements read as their complex conjugates (`TFH_VIEW_CONJ`): the lazy form of `Tensor::conj`
    /// (tenferro-tensor/src/lib.rs:622-651), taken by Contract, BatchedGemm, Permute and einsum operands.
    pub fn conj_on_load(mut self) -> Self {
        self.conj = !self.conj;
        self
    }

    /// Zero-copy `permute` (tenferro-tensor/src/lib.rs:472-487): axis `i` of the result is axis `perm[i]` of `self`.
    pub fn permute(&self, perm: &[usize]) -> Result<Self> {
        if perm.len() != self.dims.len() {
            return Err(Error::RankMismatch { expected: self.dims.len(), got: perm.len() });
        }
        let mut out = self.clone();
        for (i, &p) in perm.iter().enumerate() {
            if p >= self.dims.len() {
                return Err(Error::InvalidArgument(format!("axis {p} out of range for rank {}", self.dims.len())));
            }
            out.dims[i] = self.dims[p];
            out.strides[i] = self.strides[p];
        }
        Ok(out)
    }

    pub fn dims(&self) -> &[usize] {
        &self.dims
    }
    pub fn strides(&self) -> &[isize] {
        &self.strides
    }
    pub fn offset(&self) -> isize {
        self.offset
    }
    pub fn raw(&self) -> sys::tfh_view {
        fill_raw(self.base as *mut c_void, &self.dims, &self.strides, self.offset, if self.conj { sys::TFH_VIEW_CONJ } else { 0 })
    }
}

impl<'a, T: ScalarBase> HipViewMut<'a, T> {
    pub fn new(buffer: &'a mut HipBuffer<T>, dims: &[usize], strides: &[isize], offset: isize) -> Result<Self> {
        check_rank(dims.len())?;
        if dims.len() != strides.len() {
            return Err(Error::RankMismatch { expected: dims.len(), got: strides.len() });
        }
        Ok(Self { base: buffer.as_device_ptr(), dims: dims.to_vec(), strides: strides.to_vec(), offset, _buffer: PhantomData })
    }

    /// The whole buffer as a dense row-major tensor of shape `dims`.  Takes `&HipBuffer`: the device writes, the host
    /// borrow checker has nothing to protect; ordering between kernels is the stream's and the events' business.
    pub fn dense(buffer: &'a HipBuffer<T>, dims: &[usize]) -> Self {
        Self { base: buffer.as_device_ptr(), dims: dims.to_vec(), strides: row_major(dims), offset: 0, _buffer: PhantomData }
    }

    /// From the `StridedViewMut` that `TensorPrims::execute` is handed (device memory underneath).  The borrow of the
    /// view (`'a`) is separate from, and outlived by, the lifetime of the data it views (`'v`): `execute` passes
    /// `&mut StridedViewMut<T>` whose own lifetime parameter is invariant and unrelated to the borrow.
    pub fn from_strided<'v>(view: &'a mut StridedViewMut<'v, T>) -> Result<Self>
    where
        'v: 'a,
    {
        check_rank(view.dims().len())?;
        Ok(Self {
            base: view.data().as_ptr() as *mut T,
            dims: view.dims().to_vec(),
            strides: view.strides().to_vec(),
            offset: view.offset(),
            _buffer: PhantomData,
        })
    }

    pub fn dims(&self) -> &[usize] {
        &self.dims
    }
    pub fn strides(&self) -> &[isize] {
        &self.strides
    }
    pub fn raw(&self) -> sys::tfh_view {
        fill_raw(self.base as *mut c_void, &self.dims, &self.strides, self.offset, 0)
    }

    /// `Tensor::into_conj` (tenferro-tensor/src/lib.rs:653-658): conjugate in place.
    pub fn conj_in_place(&mut self, stream: &Stream) -> Result<()> {
        let input = self.raw();
        let mut out = self.raw();
        check(unsafe { sys::tfh_conj(dtype_tag::<T>()?, &input, &mut out, stream.raw()) })
    }

    /// `Tensor::conj` (tenferro-tensor/src/lib.rs:622-651): `self = conj(src)` elementwise, same dims.
    pub fn assign_conj(&mut self, src: &HipView<'_, T>, stream: &Stream) -> Result<()> {
        let input = src.raw();
        let mut out = self.raw();
        check(unsafe { sys::tfh_conj(dtype_tag::<T>()?, &input, &mut out, stream.raw()) })
    }
}
