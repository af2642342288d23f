//! Trait façade: the reference's `Operator` API (src/operator/mod.rs:61-99) over the rembrandt_hip C ABI.
//! Shown for Conv2dOperator::forward/backward; AffineOperator, Pool2dOperator and SoftmaxKLLossOperator
//! follow the same pattern with the entry points named in include/rembrandt_hip.h.
extern crate libc;

pub mod ffi;

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

pub struct DeviceBuffer<T> { ptr: *mut T, len: usize, ctx: Rc<DeviceContext> }

impl<T> DeviceBuffer<T> {
  pub fn zeros(len: usize, ctx: Rc<DeviceContext>) -> DeviceBuffer<T> {
    let mut p: *mut c_void = ptr::null_mut();
    unwrap(unsafe { rh_malloc(ctx.raw, len * ::std::mem::size_of::<T>(), &mut p) }, "rh_malloc");
    DeviceBuffer{ptr: p as *mut T, len: len, ctx: ctx}
  }
  pub fn as_ptr(&self) -> *const T { self.ptr }
  pub fn as_mut_ptr(&mut self) -> *mut T { self.ptr }
  pub fn len(&self) -> usize { self.len }
}

impl<T> Drop for DeviceBuffer<T> {
  fn drop(&mut self) { unsafe { rh_free(self.ctx.raw, self.ptr as *mut c_void); } }
}

pub type SharedDeviceBuf<T> = Rc<RefCell<DeviceBuffer<T>>>;

#[derive(Clone, Copy, Debug)]
pub enum ActivationFunction { Identity, Rect, Logistic, Tanh }

#[derive(Clone, Copy, Debug)]
pub enum OpPhase { Inference, Training{t: usize} }

#[derive(Clone, Copy, Debug)]
pub struct Conv2dOperatorConfig {
  pub in_dims:      (usize, usize, usize),
  pub conv_size:    usize,
  pub conv_stride:  usize,
  pub conv_pad:     usize,
  pub out_channels: usize,
  pub act_func:     ActivationFunction,
}

pub struct Conv2dOperator {
  batch_cap:  usize,
  config:     Conv2dOperatorConfig,
  context:    Rc<DeviceContext>,
  in_act:     SharedDeviceBuf<f32>,
  in_delta:   Option<SharedDeviceBuf<f32>>,
  out_act:    SharedDeviceBuf<f32>,
  out_delta:  SharedDeviceBuf<f32>,
  weights:    DeviceBuffer<f32>,
  bias:       DeviceBuffer<f32>,
  grad_weights: DeviceBuffer<f32>,
  grad_bias:  DeviceBuffer<f32>,
  workspace:  DeviceBuffer<u8>,
}

impl Conv2dOperator {
  fn geom(&self, batch_size: usize) -> rh_conv_geom {
    let (w, h, c) = self.config.in_dims;
    rh_conv_geom{n: batch_size as i32, c: c as i32, h: h as i32, w: w as i32,
                 k: self.config.out_channels as i32, r: self.config.conv_size as i32, s: self.config.conv_size as i32,
                 stride: self.config.conv_stride as i32, pad: self.config.conv_pad as i32}
  }

  /// src/operator/mod.rs:1663-1718: conv, bias add, ReLU -- one launch with the fused epilogue.
  pub fn forward(&mut self, batch_size: usize, _phase: OpPhase) {
    assert!(batch_size <= self.batch_cap);
    let g = self.geom(batch_size);
    let flags = RH_FUSE_BIAS | match self.config.act_func {
      ActivationFunction::Identity => 0,
      ActivationFunction::Rect => RH_FUSE_RELU,
      _ => unimplemented!(),
    };
    let ws_len = self.workspace.len();
    unwrap(unsafe { rh_conv2d_fwd(&g, 1.0, self.in_act.borrow().as_ptr(), self.weights.as_ptr(), 0.0,
                                  self.out_act.borrow_mut().as_mut_ptr(), self.bias.as_ptr(),
                                  self.workspace.as_mut_ptr() as *mut c_void, ws_len, flags,
                                  self.context.stream()) }, "conv2d forward");
  }

  /// src/operator/mod.rs:1720-1795: ReLU mask in place, filter and bias gradients (beta = 1), data gradient.
  pub fn backward(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    let g = self.geom(batch_size);
    let stream = self.context.stream();
    let out_len = self.out_act.borrow().len() / self.batch_cap;
    let plane = (out_len / self.config.out_channels) as i32;
    let ws_len = self.workspace.len();
    let ws = self.workspace.as_mut_ptr() as *mut c_void;
    unsafe {
      if let ActivationFunction::Rect = self.config.act_func {
        rembrandt_kernel_batch_map_rect_backprop_inplace(self.out_act.borrow().as_ptr(), out_len as i32,
                                                         batch_size as i32, self.out_delta.borrow_mut().as_mut_ptr(), stream);
        unwrap(rh_last_error(), "rect backprop");
      }
      unwrap(rh_conv2d_bwd_filter(&g, 1.0, self.in_act.borrow().as_ptr(), self.out_delta.borrow().as_ptr(), 1.0,
                                  self.grad_weights.as_mut_ptr(), ws, ws_len, 0, stream), "conv2d backward filter");
      unwrap(rh_conv2d_bwd_bias(batch_size as i32, self.config.out_channels as i32, plane, 1.0,
                                self.out_delta.borrow().as_ptr(), 1.0, self.grad_bias.as_mut_ptr(), stream),
             "conv2d backward bias");
      if let Some(ref in_delta) = self.in_delta {
        unwrap(rh_conv2d_bwd_data(&g, 1.0, self.weights.as_ptr(), self.out_delta.borrow().as_ptr(), 0.0,
                                  in_delta.borrow_mut().as_mut_ptr(), ws, ws_len, 0, stream), "conv2d backward data");
      }
    }
  }
}
