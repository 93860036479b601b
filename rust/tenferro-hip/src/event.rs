//! Streams and `CompletionEvent` (tenferro-tensor/src/lib.rs:301-309): the handle a `Tensor` keeps while the kernels
//! that produce it are still running, `Tensor::wait` / `is_ready` (:677-713) and chaining without a host wait
//! (tenferro-einsum/src/lib.rs:146-177).

use std::ffi::c_void;

use tenferro_device::Result;
use tenferro_hip_sys as sys;

use crate::check;

/// A HIP stream.  `Stream::null()` is the device's default stream; `Stream::new()` creates one (default priority)
/// and destroys it on drop.  Calls that enqueue on the same stream must not overlap in time (each stream owns
/// scratch memory that successive calls reuse in stream order); different streams may be driven from different
/// threads at once.
pub struct Stream {
    raw: sys::tfh_stream,
    owned: bool,
}

unsafe impl Send for Stream {}

impl Stream {
    pub fn null() -> Self {
        Self { raw: std::ptr::null_mut(), owned: false }
    }
    pub fn new() -> Result<Self> {
        let mut raw: sys::tfh_stream = std::ptr::null_mut();
        check(unsafe { sys::tfh_stream_create(&mut raw) })?;
        Ok(Self { raw, owned: true })
    }
    /// Wraps a `hipStream_t` the caller owns (it is not destroyed on drop).
    ///
    /// # Safety
    /// `raw` must be a live HIP stream of the current device, or null.
    pub unsafe fn from_raw(raw: *mut c_void) -> Self {
        Self { raw, owned: false }
    }
    pub fn raw(&self) -> sys::tfh_stream {
        self.raw
    }
    pub fn synchronize(&self) -> Result<()> {
        check(unsafe { sys::tfh_stream_synchronize(self.raw) })
    }
    /// Work enqueued on this stream from now on starts after `event` has completed; the host does not wait.
    pub fn wait_event(&self, event: &CompletionEvent) -> Result<()> {
        check(unsafe { sys::tfh_stream_wait_event(self.raw, event.raw) })
    }
}

impl Drop for Stream {
    fn drop(&mut self) {
        if self.owned && !self.raw.is_null() {
            unsafe { sys::tfh_stream_destroy(self.raw) };
        }
    }
}

/// Completion of everything enqueued on a stream up to the point of [`CompletionEvent::record`]
/// (tenferro-tensor/src/lib.rs:301-309 leaves the body as a placeholder "for a CUDA/HIP event handle").
pub struct CompletionEvent {
    raw: sys::tfh_event,
}

unsafe impl Send for CompletionEvent {}
unsafe impl Sync for CompletionEvent {}

impl CompletionEvent {
    /// A fresh event recorded on `stream`: what a GPU operation stores in the `event` field of its result.
    pub fn record(stream: &Stream) -> Result<Self> {
        let mut raw: sys::tfh_event = std::ptr::null_mut();
        check(unsafe { sys::tfh_event_create(&mut raw) })?;
        let event = Self { raw };
        check(unsafe { sys::tfh_event_record(event.raw, stream.raw()) })?;
        Ok(event)
    }
    /// Records again, on the same or another stream; earlier waits are unaffected.
    pub fn rerecord(&self, stream: &Stream) -> Result<()> {
        check(unsafe { sys::tfh_event_record(self.raw, stream.raw()) })
    }
    /// `Tensor::wait` (tenferro-tensor/src/lib.rs:701-704): blocks the calling thread until the event has completed.
    pub fn wait(&self) -> Result<()> {
        check(unsafe { sys::tfh_event_synchronize(self.raw) })
    }
    /// `Tensor::is_ready` (tenferro-tensor/src/lib.rs:711-713) for a tensor whose `event` is `Some`.
    pub fn is_ready(&self) -> Result<bool> {
        let mut ready = 0i32;
        check(unsafe { sys::tfh_event_query(self.raw, &mut ready) })?;
        Ok(ready != 0)
    }
}

impl Drop for CompletionEvent {
    fn drop(&mut self) {
        if !self.raw.is_null() {
            unsafe { sys::tfh_event_destroy(self.raw) };
        }
    }
}
