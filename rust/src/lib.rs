//! The reference's operator API (src/operator/mod.rs:61-99, loss.rs:20-39, worker.rs:52-76) over the
//! rembrandt_hip C ABI: device context and buffers here, the `Operator` / `LossOperator` /
//! `OperatorWorker` traits with `Conv2dOperator`, `AffineOperator`, `Pool2dOperator`,
//! `SoftmaxKLLossOperator` and `SequentialOperatorWorker` in `operator`.
//!
//! Written for the reference's toolchain (rustc 1.9 nightly, `libc`); the image this library is built and
//! tested in has no Rust toolchain, so this crate is source a maintainer adopts, and the tested boundary
//! is the C ABI it binds (include/rembrandt_hip.h), driven by the C++ mirror of the same classes.
extern crate libc;

pub mod ffi;
pub mod operator;

use ffi::*;
use std::cell::RefCell;
use std::os::raw::c_void;
use std::ptr;
use std::rc::Rc;

pub struct DeviceContext { pub raw: *mut rh_ctx }

impl DeviceContext {
  pub fn new(device_idx: usize) -> DeviceContext {
    let mut raw = ptr::null_mut();
    unwrap(unsafe { rh_ctx_create(device_idx as i32, &mut raw) }, "rh_ctx_create");
    DeviceContext{raw: raw}
  }
  pub fn stream(&self) -> rh_stream_t { unsafe { rh_ctx_stream(self.raw) } }
  pub fn sync(&self) { unwrap(unsafe { rh_ctx_sync(self.raw) }, "rh_ctx_sync"); }
}

impl Drop for DeviceContext {
  fn drop(&mut self) { unsafe { rh_ctx_destroy(self.raw); } }
}

/// `array_cuda::device::DeviceBuffer`: owned device memory with the synchronous copies the operators use.
pub struct DeviceBuffer<T> { ptr: *mut T, len: usize, ctx: Rc<DeviceContext> }

impl<T: Copy> DeviceBuffer<T> {
  pub fn zeros(len: usize, ctx: Rc<DeviceContext>) -> DeviceBuffer<T> {
    let mut p: *mut c_void = ptr::null_mut();
    let bytes = len * ::std::mem::size_of::<T>();
    unwrap(unsafe { rh_malloc(ctx.raw, bytes, &mut p) }, "rh_malloc");
    // every element type used here (f32, i32, u8) is 4-byte fillable or a byte buffer rounded up by rh_malloc
    unwrap(unsafe { rh_memset_f32(p as *mut f32, 0.0, bytes / 4, ctx.stream()) }, "rh_memset_f32");
    DeviceBuffer{ptr: p as *mut T, len: len, ctx: ctx}
  }
  pub fn as_ptr(&self) -> *const T { self.ptr }
  pub fn as_mut_ptr(&mut self) -> *mut T { self.ptr }
  pub fn len(&self) -> usize { self.len }
  pub fn context(&self) -> Rc<DeviceContext> { self.ctx.clone() }
  /// `sync_load`: host slice to device, returns when the host memory may be reused.
  pub fn sync_load(&mut self, src: &[T]) {
    assert!(src.len() <= self.len);
    let bytes = src.len() * ::std::mem::size_of::<T>();
    unwrap(unsafe { rh_load_sync(self.ctx.raw, self.ptr as *mut c_void, src.as_ptr() as *const c_void, bytes) },
           "rh_load_sync");
  }
  /// `sync_store`: device to host slice, blocking.
  pub fn sync_store(&self, dst: &mut [T]) {
    assert!(dst.len() <= self.len);
    let bytes = dst.len() * ::std::mem::size_of::<T>();
    unwrap(unsafe { rh_store_sync(self.ctx.raw, dst.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, bytes) },
           "rh_store_sync");
  }
}

impl<T> Drop for DeviceBuffer<T> {
  fn drop(&mut self) { unsafe { rh_free(self.ctx.raw, self.ptr as *mut c_void); } }
}

pub type SharedDeviceBuf<T> = Rc<RefCell<DeviceBuffer<T>>>;

pub fn shared<T: Copy>(len: usize, ctx: Rc<DeviceContext>) -> SharedDeviceBuf<T> {
  Rc::new(RefCell::new(DeviceBuffer::zeros(len, ctx)))
}
