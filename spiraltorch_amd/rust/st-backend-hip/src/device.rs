//! RAII handles over the C ABI's device memory, streams and events: what the reference's `real` module did with
//! raw `hipMalloc` / `hipStreamCreate` pairs around every call (real.rs:718-756), as owned values that callers can
//! keep between operators so that tensors stay in HBM.

use std::marker::PhantomData;
use std::os::raw::c_void;
use std::ptr;

use crate::ffi;
use crate::{status, HipErr};

/// A HIP stream; destroyed on drop.  `Stream::null()` is the default stream.
#[derive(Debug)]
pub struct Stream {
    raw: *mut c_void,
    owned: bool,
}

// The handle is an opaque pointer the HIP runtime synchronises internally.
unsafe impl Send for Stream {}

impl Stream {
    pub fn new() -> Result<Self, HipErr> {
        let mut raw = ptr::null_mut();
        status(unsafe { ffi::st_hip_stream_create(&mut raw) })?;
        Ok(Self { raw, owned: true })
    }

    pub const fn null() -> Self {
        Self { raw: ptr::null_mut(), owned: false }
    }

    pub fn synchronize(&self) -> Result<(), HipErr> {
        status(unsafe { ffi::st_hip_stream_synchronize(self.raw) })
    }

    pub fn as_raw(&self) -> *mut c_void {
        self.raw
    }
}

impl Drop for Stream {
    fn drop(&mut self) {
        if self.owned {
            unsafe { ffi::st_hip_stream_destroy(self.raw) };
        }
    }
}

/// A timing event on a stream.
#[derive(Debug)]
pub struct Event {
    raw: *mut c_void,
}

unsafe impl Send for Event {}

impl Event {
    pub fn new() -> Result<Self, HipErr> {
        let mut raw = ptr::null_mut();
        status(unsafe { ffi::st_hip_event_create(&mut raw) })?;
        Ok(Self { raw })
    }

    pub fn record(&self, stream: &Stream) -> Result<(), HipErr> {
        status(unsafe { ffi::st_hip_event_record(self.raw, stream.as_raw()) })
    }

    pub fn synchronize(&self) -> Result<(), HipErr> {
        status(unsafe { ffi::st_hip_event_synchronize(self.raw) })
    }

    /// Milliseconds from `self` to `stop`, both recorded and complete.
    pub fn elapsed_ms(&self, stop: &Event) -> Result<f32, HipErr> {
        let mut ms = 0.0f32;
        status(unsafe { ffi::st_hip_event_elapsed_ms(self.raw, stop.raw, &mut ms) })?;
        Ok(ms)
    }
}

impl Drop for Event {
    fn drop(&mut self) {
        unsafe { ffi::st_hip_event_destroy(self.raw) };
    }
}

/// `len` elements of `T` in device memory; freed on drop.
#[derive(Debug)]
pub struct DeviceBuffer<T: Copy> {
    raw: *mut c_void,
    len: usize,
    marker: PhantomData<T>,
}

unsafe impl<T: Copy + Send> Send for DeviceBuffer<T> {}

impl<T: Copy> DeviceBuffer<T> {
    pub fn new(len: usize) -> Result<Self, HipErr> {
        let bytes = len
            .checked_mul(std::mem::size_of::<T>())
            .ok_or_else(|| HipErr::Other("device buffer size overflows usize".into()))?;
        let mut raw = ptr::null_mut();
        status(unsafe { ffi::st_hip_malloc(&mut raw, bytes) })?;
        Ok(Self { raw, len, marker: PhantomData })
    }

    /// Allocates and uploads `host` (synchronous on `stream`).
    pub fn from_slice(host: &[T], stream: &Stream) -> Result<Self, HipErr> {
        let buffer = Self::new(host.len())?;
        buffer.upload(host, stream)?;
        Ok(buffer)
    }

    pub fn upload(&self, host: &[T], stream: &Stream) -> Result<(), HipErr> {
        if host.len() != self.len {
            return Err(HipErr::Other(format!("upload of {} elements into a device buffer of {}", host.len(), self.len)));
        }
        status(unsafe {
            ffi::st_hip_memcpy_h2d(self.raw, host.as_ptr() as *const c_void, std::mem::size_of_val(host), stream.as_raw())
        })
    }

    pub fn download(&self, host: &mut [T], stream: &Stream) -> Result<(), HipErr> {
        if host.len() != self.len {
            return Err(HipErr::Other(format!("download of a device buffer of {} elements into {}", self.len, host.len())));
        }
        status(unsafe {
            ffi::st_hip_memcpy_d2h(host.as_mut_ptr() as *mut c_void, self.raw, std::mem::size_of_val(host), stream.as_raw())
        })
    }

    pub fn len(&self) -> usize {
        self.len
    }

    pub fn is_empty(&self) -> bool {
        self.len == 0
    }

    pub fn as_ptr(&self) -> *const T {
        self.raw as *const T
    }

    pub fn as_mut_ptr(&mut self) -> *mut T {
        self.raw as *mut T
    }
}

impl<T: Copy> Drop for DeviceBuffer<T> {
    fn drop(&mut self) {
        unsafe { ffi::st_hip_free(self.raw) };
    }
}
