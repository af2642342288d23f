//! `Operator`, `LossOperator`, `OperatorWorker` (src/operator/mod.rs:61-99, loss.rs:20-39, worker.rs:52-76) and
//! the four operators of the hot path plus the sequential worker, each method a handful of calls into
//! include/rembrandt_hip.h.  Behaviour follows the reference: every native error panics, parameters of one
//! operator are `weights` then `bias`, gradients accumulate (beta = 1) until `reset`, and the SGD calls are the
//! BLAS-1 sequences of src/operator/mod.rs:1178-1236.  The second-generation calls (`backward_scaled`, `descend`,
//! `reset_gradients`: src/layer_new.rs:596-617, 1093-1154, src/arch_new.rs:527-552) are methods of the same trait.
//! Beyond the reference's call list the operators use the library's folded forms where they give the same values:
//! filter and bias gradient in one call, the ReLU backward mask inside the consumer's backward kernel, and the whole
//! SGD update as one multi-tensor launch (`SequentialOperatorWorker::fused_sgd_step`).
use ffi::*;
use super::{DeviceBuffer, DeviceContext, SharedDeviceBuf, shared};

use libc::{c_void};
use std::fs::{self, File};
use std::io::{Read, Write};
use std::path::{Path, PathBuf};
use std::rc::Rc;

#[derive(Clone, Copy, Debug, PartialEq)]
pub enum OpCapability { Forward, Backward }

#[derive(Clone, Copy, Debug)]
pub enum OpPhase { Inference, Training{t: usize} }

#[derive(Clone, Copy, Debug)]
pub enum Regularization { L2{l2_reg_coef: f32} }

#[derive(Clone, Copy, Debug)]
pub enum ActivationFunction { Identity, Rect, Logistic, Tanh }

#[derive(Clone, Copy, Debug)]
pub enum ParamsInit { Disabled, Uniform{half_range: f32}, Normal{std: f32}, Xavier, KaimingFwd }

#[derive(Clone, Copy, Debug, PartialEq)]
pub enum PoolOperation { Max, Average }

pub trait Operator {
  fn batch_size(&self) -> usize;
  fn get_output_vars(&self) -> Option<SharedDeviceBuf<f32>> { None }
  fn get_output_deltas(&self) -> Option<SharedDeviceBuf<f32>> { None }
  fn init_params(&mut self, _shared_seed: [u64; 2]) {}
  /// Parameter / optimizer-state blobs (src/operator/mod.rs:65-68): NdArray records, weights then bias
  /// (momentum buffers for the state); `decode_*` returns the number of bytes it consumed.
  fn decode_params(&mut self, _blob: &[u8]) -> usize { 0 }
  fn encode_params(&mut self, _blob: &mut Vec<u8>) {}
  fn decode_state(&mut self, _blob: &[u8]) -> usize { 0 }
  fn encode_state(&mut self, _blob: &mut Vec<u8>) {}
  fn forward(&mut self, batch_size: usize, phase: OpPhase);
  fn backward(&mut self, batch_size: usize);
  fn regularize(&mut self, _reg: Regularization) {}
  fn accumulate_grads(&mut self, _scale: f32, _momentum: f32) {}
  fn update_params(&mut self, _scale: f32) {}
  fn update_params2(&mut self, _grad_scale: f32, _update_scale: f32) {}
  fn save_params(&mut self) {}
  fn restore_params(&mut self) {}
  fn reset(&mut self) {}
  // second generation
  fn backward_scaled(&mut self, batch_size: usize, _scale: f32) { self.backward(batch_size); }
  fn descend(&mut self, _scale: f32, _l2_reg_coef: f32) {}
  fn reset_gradients(&mut self, _momentum: f32) {}
  /// Rows of one multi-tensor SGD launch (rh_sgd_momentum_step_multi): every parameter block of this operator.
  fn sgd_tensors(&mut self, _l2_reg_coef: f32, _out: &mut Vec<rh_sgd_tensor>) {}
  /// The operator above applies this operator's ReLU backward mask inside its own backward kernel
  /// (rh_conv2d_bwd_data_relu, rh_pool2d_bwd_relu); returns whether this operator agrees to skip its own pass.
  fn fold_activation_backward(&mut self) -> bool { false }
}

/// src/operator/mod.rs:101-109.
pub trait InputOperator: Operator {
  fn downcast(&self) -> &Operator;
  fn expose_host_frame_buf(&mut self, batch_idx: usize) -> &mut [u8];
  fn load_frames(&mut self, batch_size: usize);
  fn stage_shape(&mut self, batch_idx: usize, shape: (usize, usize, usize));
  fn preload_frame(&mut self, _batch_idx: usize) { unimplemented!(); }
  fn wait_preload_frames(&mut self, _batch_size: usize) { unimplemented!(); }
}

pub trait LossOperator: Operator {
  fn stage_label(&mut self, batch_idx: usize, category: i32);
  fn load_labels(&mut self, batch_size: usize);
  fn stage_weight(&mut self, batch_idx: usize, weight: f32);
  fn load_weights(&mut self, batch_size: usize);
  fn store_loss(&mut self, batch_size: usize) -> f32;
  fn store_output_categories(&mut self, batch_size: usize);
  fn get_output_categories(&self, batch_size: usize) -> &[i32];
  fn accuracy_count(&self, batch_size: usize) -> usize;
}

pub trait OperatorWorker: Operator {
  fn num_workers(&self) -> usize;
  fn worker_rank(&self) -> usize;
  fn shared_seed(&self) -> [u64; 2];
  fn input_operator(&mut self) -> &mut InputOperator;
  fn loss_count(&self) -> usize;
  fn loss_operator(&mut self, rank: usize) -> &mut LossOperator;
  // src/operator/worker.rs:62-72: what SgdOpt::train calls around its loop
  fn next(&mut self) {}
  fn checkpoint_params(&mut self, _t: usize, _prefix: &Path) { unimplemented!(); }
  fn checkpoint_state(&mut self, _prefix: &Path) { unimplemented!(); }
  fn can_rollback(&mut self, _prefix: &Path) -> Option<usize> { unimplemented!(); }
  fn rollback_params(&mut self, _t: Option<usize>, _prefix: &Path) { unimplemented!(); }
  fn rollback_state(&mut self, _prefix: &Path) { unimplemented!(); }
}

/// NdArray record: 'N','D',0,1; u32 rank; u64 dims (first index fastest); f32 data, all little-endian.
pub fn ndarray_serialize(out: &mut Vec<u8>, data: &[f32], dims: &[usize]) {
  out.extend_from_slice(&[b'N', b'D', 0, 1]);
  let nd = dims.len() as u32;
  for b in 0 .. 4 { out.push((nd >> (8 * b)) as u8); }
  for &d in dims.iter() { for b in 0 .. 8 { out.push(((d as u64) >> (8 * b)) as u8); } }
  assert_eq!(dims.iter().fold(1usize, |a, &d| a * d), data.len());
  for &v in data.iter() {
    let bits: u32 = unsafe { ::std::mem::transmute(v) };
    for b in 0 .. 4 { out.push((bits >> (8 * b)) as u8); }
  }
}

/// Returns (bytes consumed, dims, data); panics on a foreign or truncated record, as the reference's decoder does.
pub fn ndarray_deserialize(blob: &[u8]) -> (usize, Vec<usize>, Vec<f32>) {
  assert!(blob.len() >= 8 && blob[0] == b'N' && blob[1] == b'D' && blob[2] == 0 && blob[3] == 1, "NdArray: bad magic");
  let nd = (0 .. 4).fold(0u32, |a, b| a | (blob[4 + b] as u32) << (8 * b)) as usize;
  assert!(nd > 0 && nd <= 8 && blob.len() >= 8 + 8 * nd, "NdArray: bad rank or truncated header");
  let mut dims = Vec::with_capacity(nd);
  let mut off = 8;
  let mut count = 1usize;
  for _ in 0 .. nd {
    let d = (0 .. 8).fold(0u64, |a, b| a | (blob[off + b] as u64) << (8 * b)) as usize;
    dims.push(d);
    count *= d;
    off += 8;
  }
  assert!(blob.len() - off >= 4 * count, "NdArray: truncated data");
  let mut data = Vec::with_capacity(count);
  for i in 0 .. count {
    let bits = (0 .. 4).fold(0u32, |a, b| a | (blob[off + 4 * i + b] as u32) << (8 * b));
    data.push(unsafe { ::std::mem::transmute::<u32, f32>(bits) });
  }
  (off + 4 * count, dims, data)
}

/// weights / bias with their gradient, accumulated-gradient (momentum) and saved copies, and the update arithmetic
/// shared by the parametrised operators (src/operator/mod.rs:1178-1236 for affine, 1797-1870 for conv).
pub struct ParamTensors {
  pub weights:          DeviceBuffer<f32>,
  pub bias:             DeviceBuffer<f32>,
  pub grad_weights:     DeviceBuffer<f32>,
  pub grad_bias:        DeviceBuffer<f32>,
  pub acc_grad_weights: DeviceBuffer<f32>,
  pub acc_grad_bias:    DeviceBuffer<f32>,
  pub save_weights:     DeviceBuffer<f32>,
  pub save_bias:        DeviceBuffer<f32>,
  context: Rc<DeviceContext>,
}

fn encode_pair(blob: &mut Vec<u8>, w: &DeviceBuffer<f32>, b: &DeviceBuffer<f32>) {
  // the reference's Array2d bound of the weights: (in or R*S*C, out), first index fastest; the bias is (1, out)
  let (mut hw, mut hb) = (vec![0.0f32; w.len()], vec![0.0f32; b.len()]);
  w.context().sync();
  w.sync_store(&mut hw);
  b.sync_store(&mut hb);
  ndarray_serialize(blob, &hw, &[w.len() / b.len(), b.len()]);
  ndarray_serialize(blob, &hb, &[1, b.len()]);
}

fn decode_pair(blob: &[u8], w: &mut DeviceBuffer<f32>, b: &mut DeviceBuffer<f32>) -> usize {
  let (n0, d0, hw) = ndarray_deserialize(blob);
  assert!(d0.len() == 2 && d0[0] == w.len() / b.len() && d0[1] == b.len(), "weights blob has the wrong bound");
  w.sync_load(&hw);
  let (n1, d1, hb) = ndarray_deserialize(&blob[n0 ..]);
  assert!(d1.len() == 2 && d1[0] == 1 && d1[1] == b.len(), "bias blob has the wrong bound");
  b.sync_load(&hb);
  n0 + n1
}

fn axpy(alpha: f32, x: &DeviceBuffer<f32>, y: &mut DeviceBuffer<f32>, s: rh_stream_t) {
  assert_eq!(x.len(), y.len());
  unwrap(unsafe { rh_saxpy(x.len() as i64, alpha, x.as_ptr(), y.as_mut_ptr(), s) }, "rh_saxpy");
}

fn scal(alpha: f32, x: &mut DeviceBuffer<f32>, s: rh_stream_t) {
  unwrap(unsafe { rh_sscal(x.len() as i64, alpha, x.as_mut_ptr(), s) }, "rh_sscal");
}

fn copy(src: &DeviceBuffer<f32>, dst: &mut DeviceBuffer<f32>, s: rh_stream_t) {
  assert_eq!(src.len(), dst.len());
  unwrap(unsafe { rh_copy_d2d(dst.as_mut_ptr() as *mut c_void, src.as_ptr() as *const c_void, 4 * src.len(), s) },
         "rh_copy_d2d");
}

impl ParamTensors {
  pub fn new(weights_len: usize, bias_len: usize, context: Rc<DeviceContext>) -> ParamTensors {
    let w = || DeviceBuffer::zeros(weights_len, context.clone());
    let b = || DeviceBuffer::zeros(bias_len, context.clone());
    ParamTensors{
      weights: w(), bias: b(), grad_weights: w(), grad_bias: b(), acc_grad_weights: w(), acc_grad_bias: b(),
      save_weights: w(), save_bias: b(), context: context.clone(),
    }
  }

  /// The library's own documented generator (the reference's random stream lives in crates outside its tree).
  pub fn init(&mut self, init: ParamsInit, seed: [u64; 2], fan_in: usize, fan_out: usize) {
    let n = self.weights.len();
    let mut w = vec![0.0f32; n];
    match init {
      ParamsInit::Disabled => panic!("params init explicitly disabled"),
      ParamsInit::Uniform{half_range} =>
        unwrap(unsafe { rh_rng_fill_uniform(seed[0], seed[1], w.as_mut_ptr(), n, -half_range, half_range) }, "rh_rng_fill_uniform"),
      ParamsInit::Normal{std} =>
        unwrap(unsafe { rh_rng_fill_normal(seed[0], seed[1], w.as_mut_ptr(), n, 0.0, std) }, "rh_rng_fill_normal"),
      ParamsInit::Xavier => {
        let h = (6.0 / (fan_in + fan_out) as f64).sqrt() as f32;
        unwrap(unsafe { rh_rng_fill_uniform(seed[0], seed[1], w.as_mut_ptr(), n, -h, h) }, "rh_rng_fill_uniform")
      }
      ParamsInit::KaimingFwd => {
        let sd = (2.0 / fan_in as f64).sqrt() as f32;
        unwrap(unsafe { rh_rng_fill_normal(seed[0], seed[1], w.as_mut_ptr(), n, 0.0, sd) }, "rh_rng_fill_normal")
      }
    }
    self.weights.sync_load(&w);
    let b = vec![0.0f32; self.bias.len()];
    self.bias.sync_load(&b);
  }

  /// grad += l2 * params; nothing is launched for l2 == 0 (src/operator/mod.rs:1185), so a non-finite weight does
  /// not leak 0 * inf into the gradient.
  pub fn regularize(&mut self, reg: Regularization) {
    let s = self.context.stream();
    let Regularization::L2{l2_reg_coef} = reg;
    assert!(l2_reg_coef >= 0.0);
    if l2_reg_coef > 0.0 {
      axpy(l2_reg_coef, &self.weights, &mut self.grad_weights, s);
      axpy(l2_reg_coef, &self.bias, &mut self.grad_bias, s);
    }
  }
  pub fn encode_params(&self, blob: &mut Vec<u8>) { encode_pair(blob, &self.weights, &self.bias); }
  pub fn decode_params(&mut self, blob: &[u8]) -> usize { decode_pair(blob, &mut self.weights, &mut self.bias) }
  pub fn encode_state(&self, blob: &mut Vec<u8>) { encode_pair(blob, &self.acc_grad_weights, &self.acc_grad_bias); }
  pub fn decode_state(&mut self, blob: &[u8]) -> usize {
    decode_pair(blob, &mut self.acc_grad_weights, &mut self.acc_grad_bias)
  }
  /// This block's two rows of a multi-tensor SGD launch.  keep_grad = 0: the launch zeroes the gradients, which is
  /// the reference's `reset`, so a raw gradient pointer read afterwards shows zeros.
  pub fn sgd_tensors(&mut self, l2: f32, out: &mut Vec<rh_sgd_tensor>) {
    out.push(rh_sgd_tensor{w: self.weights.as_mut_ptr(), g: self.grad_weights.as_mut_ptr(),
                           v: self.acc_grad_weights.as_mut_ptr(), n: self.weights.len() as i64, l2: l2, keep_grad: 0});
    out.push(rh_sgd_tensor{w: self.bias.as_mut_ptr(), g: self.grad_bias.as_mut_ptr(),
                           v: self.acc_grad_bias.as_mut_ptr(), n: self.bias.len() as i64, l2: l2, keep_grad: 0});
  }
  /// acc = momentum * acc + scale * grad
  pub fn accumulate_grads(&mut self, scale: f32, momentum: f32) {
    let s = self.context.stream();
    scal(momentum, &mut self.acc_grad_weights, s);
    scal(momentum, &mut self.acc_grad_bias, s);
    axpy(scale, &self.grad_weights, &mut self.acc_grad_weights, s);
    axpy(scale, &self.grad_bias, &mut self.acc_grad_bias, s);
  }
  /// params += scale * acc
  pub fn update_params(&mut self, scale: f32) {
    let s = self.context.stream();
    axpy(scale, &self.acc_grad_weights, &mut self.weights, s);
    axpy(scale, &self.acc_grad_bias, &mut self.bias, s);
  }
  /// params += grad_scale * grad + update_scale * acc
  pub fn update_params2(&mut self, grad_scale: f32, update_scale: f32) {
    let s = self.context.stream();
    if grad_scale != 0.0 {
      axpy(grad_scale, &self.grad_weights, &mut self.weights, s);
      axpy(grad_scale, &self.grad_bias, &mut self.bias, s);
    }
    if update_scale != 0.0 {
      axpy(update_scale, &self.acc_grad_weights, &mut self.weights, s);
      axpy(update_scale, &self.acc_grad_bias, &mut self.bias, s);
    }
  }
  pub fn save_params(&mut self) {
    let s = self.context.stream();
    copy(&self.weights, &mut self.save_weights, s);
    copy(&self.bias, &mut self.save_bias, s);
  }
  pub fn restore_params(&mut self) {
    let s = self.context.stream();
    copy(&self.save_weights, &mut self.weights, s);
    copy(&self.save_bias, &mut self.bias, s);
  }
  /// grad = 0
  pub fn reset(&mut self) {
    let s = self.context.stream();
    unwrap(unsafe { rh_memset_f32(self.grad_weights.as_mut_ptr(), 0.0, self.grad_weights.len(), s) }, "rh_memset_f32");
    unwrap(unsafe { rh_memset_f32(self.grad_bias.as_mut_ptr(), 0.0, self.grad_bias.len(), s) }, "rh_memset_f32");
  }
  /// Second generation: grad += l2 * params; params -= scale * grad (the gradient buffer is the velocity).
  pub fn descend(&mut self, scale: f32, l2_reg_coef: f32) {
    let s = self.context.stream();
    unwrap(unsafe { rh_descend(self.weights.len() as i64, self.weights.as_mut_ptr(), self.grad_weights.as_mut_ptr(),
                               scale, l2_reg_coef, s) }, "rh_descend");
    unwrap(unsafe { rh_descend(self.bias.len() as i64, self.bias.as_mut_ptr(), self.grad_bias.as_mut_ptr(),
                               scale, l2_reg_coef, s) }, "rh_descend");
  }
  /// Second generation: grad *= momentum.
  pub fn reset_gradients(&mut self, momentum: f32) {
    let s = self.context.stream();
    scal(momentum, &mut self.grad_weights, s);
    scal(momentum, &mut self.grad_bias, s);
  }
}

fn fuse_flags(act: ActivationFunction) -> i32 {
  RH_FUSE_BIAS | match act {
    ActivationFunction::Identity => 0,
    ActivationFunction::Rect => RH_FUSE_RELU,
    _ => unimplemented!(),
  }
}

fn rect_backprop(act: ActivationFunction, out_act: &SharedDeviceBuf<f32>, out_delta: &SharedDeviceBuf<f32>,
                 frame_len: usize, batch_size: usize, s: rh_stream_t) {
  match act {
    ActivationFunction::Identity => {}
    ActivationFunction::Rect => unsafe {
      rembrandt_kernel_batch_map_rect_backprop_inplace(out_act.borrow().as_ptr(), frame_len as i32, batch_size as i32,
                                                       out_delta.borrow_mut().as_mut_ptr(), s);
      unwrap(rh_last_error(), "rect backprop");
    },
    _ => unimplemented!(),
  }
}

// ---- Conv2dOperator (src/operator/mod.rs:1366-1870) ------------------------------------------------------------

/// The reference's algorithm selectors (src/operator/mod.rs:1366-1377).  They name cuDNN algorithms; this library
/// chooses its kernel per geometry, so both fields are accepted and ignored (the reference itself never reads
/// `bwd_backend`).  Every choice here is deterministic, which is what `CudnnDeterministic` asks for.
#[derive(Clone, Copy, Debug)]
pub enum Conv2dFwdBackend {
  CudnnFastest,
  CudnnImplicitPrecompGemm,
  CudnnFftTiling,
}

#[derive(Clone, Copy, Debug)]
pub enum Conv2dBwdBackend {
  CudnnFastest,
  CudnnDeterministic,
}

#[derive(Clone, Copy, Debug)]
pub struct Conv2dOperatorConfig {
  pub in_dims:      (usize, usize, usize),   // (width, height, channels)
  pub conv_size:    usize,
  pub conv_stride:  usize,
  pub conv_pad:     usize,
  pub out_channels: usize,
  pub act_func:     ActivationFunction,
  pub init_weights: ParamsInit,
  pub fwd_backend:  Conv2dFwdBackend,
  pub bwd_backend:  Conv2dBwdBackend,
}

impl Conv2dOperatorConfig {
  pub fn get_out_dims(&self) -> (usize, usize, usize) {
    let (w, h, _) = self.in_dims;
    let o = |x: usize| unsafe {
      rh_conv2d_out_dim(x as i32, self.conv_size as i32, self.conv_stride as i32, self.conv_pad as i32) as usize
    };
    (o(w), o(h), self.out_channels)
  }
  pub fn params_len(&self) -> usize {
    self.conv_size * self.conv_size * self.in_dims.2 * self.out_channels + self.out_channels
  }
}

pub struct Conv2dOperator {
  batch_cap:  usize,
  config:     Conv2dOperatorConfig,
  context:    Rc<DeviceContext>,
  in_act:     SharedDeviceBuf<f32>,
  in_delta:   Option<SharedDeviceBuf<f32>>,
  out_act:    SharedDeviceBuf<f32>,
  out_delta:  SharedDeviceBuf<f32>,
  params:     ParamTensors,
  backward:   bool,
  workspace:  DeviceBuffer<u8>,
  act_bwd_folded: bool,   // the operator above applies this operator's ReLU backward mask
  fold_prev_relu: bool,   // this operator's data gradient applies the ReLU backward mask of the operator below
}

impl Conv2dOperator {
  pub fn new(batch_size: usize, capability: OpCapability, config: Conv2dOperatorConfig, prev_op: &mut Operator,
             context: Rc<DeviceContext>) -> Conv2dOperator {
    let (ow, oh, oc) = config.get_out_dims();
    let out_len = ow * oh * oc * batch_size;
    let mut op = Conv2dOperator{
      batch_cap: batch_size, config: config, context: context.clone(),
      in_act: prev_op.get_output_vars().expect("Conv2dOperator missing required prev operator output vars"),
      in_delta: prev_op.get_output_deltas(),
      out_act: shared(out_len, context.clone()),
      out_delta: shared(out_len, context.clone()),
      params: ParamTensors::new(config.params_len() - config.out_channels, config.out_channels, context.clone()),
      backward: capability == OpCapability::Backward,
      workspace: DeviceBuffer::zeros(0, context.clone()),
      act_bwd_folded: false, fold_prev_relu: false,
    };
    let g = op.geom(batch_size);
    let mut ws = unsafe { rh_conv2d_workspace_bytes_upto(&g, RH_CONV_FWD) };
    if op.backward {
      ws = ::std::cmp::max(ws, unsafe { rh_conv2d_workspace_bytes_upto(&g, RH_CONV_BWD_FILTER) });
      ws = ::std::cmp::max(ws, unsafe { rh_conv2d_workspace_bytes_upto(&g, RH_CONV_BWD_DATA) });
      ws = ::std::cmp::max(ws, unsafe { rh_conv2d_bwd_bias_workspace_bytes_upto(g.n, g.k, (ow * oh) as i32) });
      if op.in_delta.is_some() && unsafe { rh_conv2d_bwd_data_relu_supported(&g) } != 0 {
        op.fold_prev_relu = prev_op.fold_activation_backward();
      }
    }
    op.workspace = DeviceBuffer::zeros(ws, context);
    op
  }

  fn geom(&self, batch_size: usize) -> rh_conv_geom {
    let (w, h, c) = self.config.in_dims;
    rh_conv_geom{n: batch_size as i32, c: c as i32, h: h as i32, w: w as i32,
                 k: self.config.out_channels as i32, r: self.config.conv_size as i32, s: self.config.conv_size as i32,
                 stride: self.config.conv_stride as i32, pad: self.config.conv_pad as i32}
  }

  fn backward_with(&mut self, batch_size: usize, scale: f32) {
    assert!(self.backward, "backward requires the Backward capability");
    assert!(batch_size <= self.batch_cap);
    let g = self.geom(batch_size);
    let stream = self.context.stream();
    let frame_len = self.out_act.borrow().len() / self.batch_cap;
    if !self.act_bwd_folded {
      rect_backprop(self.config.act_func, &self.out_act, &self.out_delta, frame_len, batch_size, stream);
    }
    let ws_len = self.workspace.len();
    let ws = self.workspace.as_mut_ptr() as *mut c_void;
    unsafe {
      // filter and bias gradient in one call (out_delta is read once where the filter gradient copies it anyway)
      unwrap(rh_conv2d_bwd_filter_bias(&g, scale, self.in_act.borrow().as_ptr(), self.out_delta.borrow().as_ptr(), 1.0,
                                       self.params.grad_weights.as_mut_ptr(), self.params.grad_bias.as_mut_ptr(),
                                       ws, ws_len, 0, stream), "conv2d backward filter / bias");
      if let Some(ref in_delta) = self.in_delta {
        if self.fold_prev_relu {
          // in_act is the output of the ReLU below: its backward mask is applied as the data gradient is written
          unwrap(rh_conv2d_bwd_data_relu(&g, 1.0, self.params.weights.as_ptr(), self.out_delta.borrow().as_ptr(), 0.0,
                                         in_delta.borrow_mut().as_mut_ptr(), self.in_act.borrow().as_ptr(), ws, ws_len,
                                         0, stream), "conv2d backward data");
        } else {
          unwrap(rh_conv2d_bwd_data(&g, 1.0, self.params.weights.as_ptr(), self.out_delta.borrow().as_ptr(), 0.0,
                                    in_delta.borrow_mut().as_mut_ptr(), ws, ws_len, 0, stream), "conv2d backward data");
        }
      }
    }
  }
}

impl Operator for Conv2dOperator {
  fn batch_size(&self) -> usize { self.batch_cap }
  fn get_output_vars(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_act.clone()) }
  fn get_output_deltas(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_delta.clone()) }
  fn init_params(&mut self, shared_seed: [u64; 2]) {
    let fan_in = self.config.conv_size * self.config.conv_size * self.config.in_dims.2;
    match self.config.init_weights {
      ParamsInit::Xavier => panic!("Conv2dOperator: Xavier init is unimplemented for this operator"),
      init => self.params.init(init, shared_seed, fan_in, self.config.out_channels),
    }
  }
  /// conv, bias add, activation: one launch (bias and ReLU in the epilogue of the contraction).
  fn forward(&mut self, batch_size: usize, _phase: OpPhase) {
    assert!(batch_size <= self.batch_cap);
    let g = self.geom(batch_size);
    let ws_len = self.workspace.len();
    unwrap(unsafe { rh_conv2d_fwd(&g, 1.0, self.in_act.borrow().as_ptr(), self.params.weights.as_ptr(), 0.0,
                                  self.out_act.borrow_mut().as_mut_ptr(), self.params.bias.as_ptr(),
                                  self.workspace.as_mut_ptr() as *mut c_void, ws_len, fuse_flags(self.config.act_func),
                                  self.context.stream()) }, "conv2d forward");
  }
  /// activation mask in place, filter and bias gradients (accumulating), data gradient.
  fn backward(&mut self, batch_size: usize) { self.backward_with(batch_size, 1.0); }
  fn backward_scaled(&mut self, batch_size: usize, scale: f32) { self.backward_with(batch_size, scale); }
  fn regularize(&mut self, reg: Regularization) { self.params.regularize(reg); }
  fn accumulate_grads(&mut self, scale: f32, momentum: f32) { self.params.accumulate_grads(scale, momentum); }
  fn update_params(&mut self, scale: f32) { self.params.update_params(scale); }
  fn update_params2(&mut self, g: f32, u: f32) { self.params.update_params2(g, u); }
  fn save_params(&mut self) { self.params.save_params(); }
  fn restore_params(&mut self) { self.params.restore_params(); }
  fn reset(&mut self) { self.params.reset(); }
  fn descend(&mut self, scale: f32, l2: f32) { self.params.descend(scale, l2); }
  fn reset_gradients(&mut self, momentum: f32) { self.params.reset_gradients(momentum); }
  fn decode_params(&mut self, blob: &[u8]) -> usize { self.params.decode_params(blob) }
  fn encode_params(&mut self, blob: &mut Vec<u8>) { self.params.encode_params(blob); }
  fn decode_state(&mut self, blob: &[u8]) -> usize { self.params.decode_state(blob) }
  fn encode_state(&mut self, blob: &mut Vec<u8>) { self.params.encode_state(blob); }
  fn sgd_tensors(&mut self, l2: f32, out: &mut Vec<rh_sgd_tensor>) { self.params.sgd_tensors(l2, out); }
  fn fold_activation_backward(&mut self) -> bool {
    match self.config.act_func {
      ActivationFunction::Rect => { self.act_bwd_folded = true; true }
      _ => false,
    }
  }
}

// ---- AffineOperator (src/operator/mod.rs:1029-1236) ------------------------------------------------------------

#[derive(Clone, Copy, Debug)]
pub struct AffineOperatorConfig {
  pub in_channels:  usize,
  pub out_channels: usize,
  pub act_func:     ActivationFunction,
  pub init_weights: ParamsInit,
}

impl AffineOperatorConfig {
  pub fn params_len(&self) -> usize { self.in_channels * self.out_channels + self.out_channels }
}

pub struct AffineOperator {
  batch_cap:  usize,
  config:     AffineOperatorConfig,
  context:    Rc<DeviceContext>,
  in_act:     SharedDeviceBuf<f32>,
  in_delta:   Option<SharedDeviceBuf<f32>>,
  out_act:    SharedDeviceBuf<f32>,
  out_delta:  SharedDeviceBuf<f32>,
  params:     ParamTensors,
  backward:   bool,
  workspace:  DeviceBuffer<u8>,
}

impl AffineOperator {
  pub fn new(batch_size: usize, capability: OpCapability, config: AffineOperatorConfig, prev_op: &Operator,
             context: Rc<DeviceContext>) -> AffineOperator {
    let (i, o, b) = (config.in_channels as i32, config.out_channels as i32, batch_size as i32);
    let backward = capability == OpCapability::Backward;
    let mut ws = unsafe { rh_sgemm_workspace_bytes_upto(o, b, i, 1) };
    if backward {
      ws = ::std::cmp::max(ws, unsafe { rh_sgemm_workspace_bytes_upto(i, o, b, 2) });
      ws = ::std::cmp::max(ws, unsafe { rh_sgemm_workspace_bytes_upto(i, b, o, 1) });
    }
    AffineOperator{
      batch_cap: batch_size, config: config, context: context.clone(),
      in_act: prev_op.get_output_vars().expect("AffineOperator missing required prev operator output vars"),
      in_delta: prev_op.get_output_deltas(),
      out_act: shared(config.out_channels * batch_size, context.clone()),
      out_delta: shared(config.out_channels * batch_size, context.clone()),
      params: ParamTensors::new(config.in_channels * config.out_channels, config.out_channels, context.clone()),
      backward: backward,
      workspace: DeviceBuffer::zeros(ws, context),
    }
  }
}

impl Operator for AffineOperator {
  fn batch_size(&self) -> usize { self.batch_cap }
  fn get_output_vars(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_act.clone()) }
  fn get_output_deltas(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_delta.clone()) }
  fn init_params(&mut self, shared_seed: [u64; 2]) {
    self.params.init(self.config.init_weights, shared_seed, self.config.in_channels, self.config.out_channels);
  }
  /// out_act(out, B) = weights(in, out)^T in_act(in, B) + bias, activation: one launch.
  fn forward(&mut self, batch_size: usize, _phase: OpPhase) {
    assert!(batch_size <= self.batch_cap);
    let (i, o, b) = (self.config.in_channels as i32, self.config.out_channels as i32, batch_size as i32);
    let ws_len = self.workspace.len();
    unwrap(unsafe { rh_sgemm_bias_act(1, 0, o, b, i, 1.0, self.params.weights.as_ptr(), i, self.in_act.borrow().as_ptr(), i,
                                      0.0, self.out_act.borrow_mut().as_mut_ptr(), o, self.params.bias.as_ptr(),
                                      self.workspace.as_mut_ptr() as *mut c_void, ws_len, fuse_flags(self.config.act_func),
                                      self.context.stream()) }, "matrix_prod");
  }
  /// grad_weights(in, out) += in_act out_delta^T; grad_bias += column sums of out_delta; in_delta = weights out_delta.
  fn backward(&mut self, batch_size: usize) {
    assert!(self.backward, "backward requires the Backward capability");
    assert!(batch_size <= self.batch_cap);
    let (i, o, b) = (self.config.in_channels as i32, self.config.out_channels as i32, batch_size as i32);
    let s = self.context.stream();
    rect_backprop(self.config.act_func, &self.out_act, &self.out_delta, self.config.out_channels, batch_size, s);
    let ws_len = self.workspace.len();
    let ws = self.workspace.as_mut_ptr() as *mut c_void;
    unsafe {
      unwrap(rh_sgemm(0, 1, i, o, b, 1.0, self.in_act.borrow().as_ptr(), i, self.out_delta.borrow().as_ptr(), o, 1.0,
                      self.params.grad_weights.as_mut_ptr(), i, ws, ws_len, 0, s), "matrix_prod");
      unwrap(rh_conv2d_bwd_bias(b, o, 1, 1.0, self.out_delta.borrow().as_ptr(), 1.0, self.params.grad_bias.as_mut_ptr(), s),
             "matrix_prod");
      if let Some(ref in_delta) = self.in_delta {
        unwrap(rh_sgemm(0, 0, i, b, o, 1.0, self.params.weights.as_ptr(), i, self.out_delta.borrow().as_ptr(), o, 0.0,
                        in_delta.borrow_mut().as_mut_ptr(), i, ws, ws_len, 0, s), "matrix_prod");
      }
    }
  }
  fn regularize(&mut self, reg: Regularization) { self.params.regularize(reg); }
  fn accumulate_grads(&mut self, scale: f32, momentum: f32) { self.params.accumulate_grads(scale, momentum); }
  fn update_params(&mut self, scale: f32) { self.params.update_params(scale); }
  fn update_params2(&mut self, g: f32, u: f32) { self.params.update_params2(g, u); }
  fn save_params(&mut self) { self.params.save_params(); }
  fn restore_params(&mut self) { self.params.restore_params(); }
  fn reset(&mut self) { self.params.reset(); }
  // AffineLayer::backward accumulates both gradients with factor 1.0 whatever `scale` is (src/layer_new.rs:583-584):
  // the inherited backward_scaled.
  fn descend(&mut self, scale: f32, l2: f32) { self.params.descend(scale, l2); }
  fn reset_gradients(&mut self, momentum: f32) { self.params.reset_gradients(momentum); }
  fn decode_params(&mut self, blob: &[u8]) -> usize { self.params.decode_params(blob) }
  fn encode_params(&mut self, blob: &mut Vec<u8>) { self.params.encode_params(blob); }
  fn decode_state(&mut self, blob: &[u8]) -> usize { self.params.decode_state(blob) }
  fn encode_state(&mut self, blob: &mut Vec<u8>) { self.params.encode_state(blob); }
  fn sgd_tensors(&mut self, l2: f32, out: &mut Vec<rh_sgd_tensor>) { self.params.sgd_tensors(l2, out); }
}

// ---- Pool2dOperator (src/operator/mod.rs:1990-2125) ------------------------------------------------------------

#[derive(Clone, Copy, Debug)]
pub struct Pool2dOperatorConfig {
  pub in_dims:      (usize, usize, usize),
  pub pool_size:    usize,
  pub pool_stride:  usize,
  pub pool_pad:     usize,
  pub pool_op:      PoolOperation,
}

impl Pool2dOperatorConfig {
  pub fn get_out_dims(&self) -> (usize, usize, usize) {
    let (w, h, c) = self.in_dims;
    let o = |x: usize| unsafe {
      rh_pool2d_out_dim(x as i32, self.pool_size as i32, self.pool_stride as i32, self.pool_pad as i32, 0) as usize
    };
    (o(w), o(h), c)
  }
}

pub struct Pool2dOperator {
  batch_cap:  usize,
  config:     Pool2dOperatorConfig,
  context:    Rc<DeviceContext>,
  in_act:     SharedDeviceBuf<f32>,
  in_delta:   Option<SharedDeviceBuf<f32>>,
  out_act:    SharedDeviceBuf<f32>,
  out_delta:  SharedDeviceBuf<f32>,
  argmax:     DeviceBuffer<i32>,   // which input element each max window took: makes the backward pass a scatter
  fold_relu:  bool,                // backward also applies the ReLU backward mask of the operator below
}

impl Pool2dOperator {
  pub fn new(batch_size: usize, config: Pool2dOperatorConfig, prev_op: &mut Operator, context: Rc<DeviceContext>) -> Pool2dOperator {
    let (ow, oh, oc) = config.get_out_dims();
    let out_len = ow * oh * oc * batch_size;
    let mut op = Pool2dOperator{
      batch_cap: batch_size, config: config, context: context.clone(),
      in_act: prev_op.get_output_vars().expect("Pool2dOperator missing required prev operator output vars"),
      in_delta: prev_op.get_output_deltas(),
      out_act: shared(out_len, context.clone()),
      out_delta: shared(out_len, context.clone()),
      argmax: DeviceBuffer::zeros(out_len, context),
      fold_relu: false,
    };
    let g = op.geom(batch_size);
    match config.pool_op {
      PoolOperation::Max => {
        if op.in_delta.is_some() && unsafe { rh_pool2d_bwd_relu_supported(&g) } != 0 {
          op.fold_relu = prev_op.fold_activation_backward();
        }
      }
      // average pooling: the same fold with the pool's input (the ReLU's output) as the mask
      PoolOperation::Average => {
        if op.in_delta.is_some() { op.fold_relu = prev_op.fold_activation_backward(); }
      }
    }
    op
  }
  fn geom(&self, batch_size: usize) -> rh_pool_geom {
    let (w, h, c) = self.config.in_dims;
    rh_pool_geom{n: batch_size as i32, c: c as i32, h: h as i32, w: w as i32, size: self.config.pool_size as i32,
                 stride: self.config.pool_stride as i32, pad: self.config.pool_pad as i32,
                 mode: match self.config.pool_op { PoolOperation::Max => 0, PoolOperation::Average => 1 }, round: 0}
  }
}

impl Operator for Pool2dOperator {
  fn batch_size(&self) -> usize { self.batch_cap }
  fn get_output_vars(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_act.clone()) }
  fn get_output_deltas(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_delta.clone()) }
  fn forward(&mut self, batch_size: usize, _phase: OpPhase) {
    assert!(batch_size <= self.batch_cap);
    let g = self.geom(batch_size);
    unwrap(unsafe { rh_pool2d_fwd(&g, self.in_act.borrow().as_ptr(), self.out_act.borrow_mut().as_mut_ptr(),
                                  self.argmax.as_mut_ptr(), self.context.stream()) }, "pool2d forward");
  }
  fn backward(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    let g = self.geom(batch_size);
    if let Some(ref in_delta) = self.in_delta {
      if self.fold_relu && self.config.pool_op == PoolOperation::Average {
        unwrap(unsafe { rh_pool2d_bwd_avg_relu(&g, self.in_act.borrow().as_ptr(), self.out_delta.borrow().as_ptr(),
                                               in_delta.borrow_mut().as_mut_ptr(), self.context.stream()) }, "pool2d backward");
      } else if self.fold_relu {
        // an arg-max element carries x = y, so windows with y <= 0 route nothing: the ReLU mask without a pass of its own
        unwrap(unsafe { rh_pool2d_bwd_relu(&g, self.out_act.borrow().as_ptr(), self.out_delta.borrow().as_ptr(),
                                           in_delta.borrow_mut().as_mut_ptr(), self.argmax.as_ptr(),
                                           self.context.stream()) }, "pool2d backward");
      } else {
        unwrap(unsafe { rh_pool2d_bwd(&g, self.in_act.borrow().as_ptr(), self.out_act.borrow().as_ptr(),
                                      self.out_delta.borrow().as_ptr(), in_delta.borrow_mut().as_mut_ptr(),
                                      self.argmax.as_ptr(), self.context.stream()) }, "pool2d backward");
      }
    }
  }
}

// ---- SoftmaxKLLossOperator (src/operator/loss.rs:41-260) -------------------------------------------------------

#[derive(Clone, Copy, Debug)]
pub struct CategoricalLossConfig {
  pub num_categories: usize,
}

pub struct SoftmaxKLLossOperator {
  batch_cap:    usize,
  loss_config:  CategoricalLossConfig,
  context:      Rc<DeviceContext>,
  in_act:       SharedDeviceBuf<f32>,
  in_delta:     SharedDeviceBuf<f32>,
  label_cats:   DeviceBuffer<i32>,
  label_cats_h: Vec<i32>,
  weights:      DeviceBuffer<f32>,
  weights_h:    Vec<f32>,
  out_values:   DeviceBuffer<f32>,
  max_value:    DeviceBuffer<f32>,
  out_cats:     DeviceBuffer<i32>,
  out_cats_h:   Vec<i32>,
  out_loss1:    DeviceBuffer<f32>,
  out_loss:     DeviceBuffer<f32>,
}

impl SoftmaxKLLossOperator {
  pub fn new(batch_size: usize, loss_config: CategoricalLossConfig, prev_op: &Operator, context: Rc<DeviceContext>)
      -> SoftmaxKLLossOperator {
    let c = || context.clone();
    SoftmaxKLLossOperator{
      batch_cap: batch_size, loss_config: loss_config, context: c(),
      in_act: prev_op.get_output_vars().expect("SoftmaxKLLossOperator missing required prev operator output vars"),
      in_delta: prev_op.get_output_deltas().expect("SoftmaxKLLossOperator missing required prev operator output deltas"),
      label_cats: DeviceBuffer::zeros(batch_size, c()), label_cats_h: vec![0; batch_size],
      weights: DeviceBuffer::zeros(batch_size, c()), weights_h: vec![0.0; batch_size],
      out_values: DeviceBuffer::zeros(loss_config.num_categories * batch_size, c()),
      max_value: DeviceBuffer::zeros(batch_size, c()),
      out_cats: DeviceBuffer::zeros(batch_size, c()), out_cats_h: vec![0; batch_size],
      out_loss1: DeviceBuffer::zeros(batch_size, c()), out_loss: DeviceBuffer::zeros(1, c()),
    }
  }
}

impl Operator for SoftmaxKLLossOperator {
  fn batch_size(&self) -> usize { self.batch_cap }
  fn forward(&mut self, batch_size: usize, _phase: OpPhase) {
    assert!(batch_size <= self.batch_cap);
    unwrap(unsafe { rh_softmax_fwd(self.in_act.borrow().as_ptr(), self.out_values.as_mut_ptr(),
                                   self.loss_config.num_categories as i32, batch_size as i32, self.context.stream()) },
           "softmax forward");
  }
  fn backward(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    unsafe {
      rembrandt_kernel_batch_map_softmax_kl_backward(self.out_values.as_ptr(), self.loss_config.num_categories as i32,
                                                     batch_size as i32, self.label_cats.as_ptr(), self.weights.as_ptr(),
                                                     self.in_delta.borrow_mut().as_mut_ptr(), self.context.stream());
      unwrap(rh_last_error(), "softmax_kl_backward");
    }
  }
}

impl LossOperator for SoftmaxKLLossOperator {
  fn stage_label(&mut self, batch_idx: usize, category: i32) {
    assert!(batch_idx < self.batch_cap);
    assert!(category >= 0 && (category as usize) < self.loss_config.num_categories);
    self.label_cats_h[batch_idx] = category;
  }
  fn load_labels(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    self.label_cats.sync_load(&self.label_cats_h);
  }
  fn stage_weight(&mut self, batch_idx: usize, weight: f32) {
    assert!(batch_idx < self.batch_cap);
    self.weights_h[batch_idx] = weight;
  }
  fn load_weights(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    self.weights.sync_load(&self.weights_h);
  }
  fn store_loss(&mut self, batch_size: usize) -> f32 {
    assert!(batch_size <= self.batch_cap);
    let s = self.context.stream();
    unsafe {
      rembrandt_kernel_batch_map_softmax_kl_loss1(self.out_values.as_ptr(), self.loss_config.num_categories as i32,
                                                  batch_size as i32, self.label_cats.as_ptr(), self.weights.as_ptr(), 0.0,
                                                  self.out_loss1.as_mut_ptr(), s);
      unwrap(rh_last_error(), "softmax_kl_loss1");
      rembrandt_kernel_batch_blockreduce_sum(self.out_loss1.as_ptr(), batch_size as i32, 1, self.out_loss.as_mut_ptr(), 0.0, s);
      unwrap(rh_last_error(), "blockreduce_sum");
    }
    let mut h = [0.0f32];
    self.out_loss.sync_store(&mut h);
    h[0]
  }
  fn store_output_categories(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    unsafe {
      rembrandt_kernel_batch_blockreduce_argmax(self.out_values.as_ptr(), self.loss_config.num_categories as i32,
                                                batch_size as i32, self.max_value.as_mut_ptr(), self.out_cats.as_mut_ptr(),
                                                self.context.stream());
      unwrap(rh_last_error(), "blockreduce_argmax");
    }
    self.out_cats.sync_store(&mut self.out_cats_h);
  }
  fn get_output_categories(&self, batch_size: usize) -> &[i32] { &self.out_cats_h[ .. batch_size] }
  fn accuracy_count(&self, batch_size: usize) -> usize {
    (0 .. batch_size).filter(|&i| self.label_cats_h[i] == self.out_cats_h[i]).count()
  }
}

// ---- input + SequentialOperatorWorker (src/operator/worker.rs:100-480) -----------------------------------------

/// The head of a chain (`Data3dOperator` without preprocessing, src/operator/mod.rs:507-640): u8 frames are staged in
/// host memory, copied to the device and cast to f32 (`normalize`: divided by 255), or loaded as f32 directly.
pub struct FrameInputOperator {
  batch_cap: usize,
  frame_len: usize,
  normalize: bool,
  context:   Rc<DeviceContext>,
  in_buf_h:  Vec<u8>,
  in_buf:    DeviceBuffer<u8>,
  out_act:   SharedDeviceBuf<f32>,
}

impl FrameInputOperator {
  pub fn new(batch_size: usize, frame_len: usize, normalize: bool, context: Rc<DeviceContext>) -> FrameInputOperator {
    FrameInputOperator{batch_cap: batch_size, frame_len: frame_len, normalize: normalize, context: context.clone(),
                       in_buf_h: vec![0u8; frame_len * batch_size],
                       in_buf: DeviceBuffer::zeros(frame_len * batch_size, context.clone()),
                       out_act: shared(frame_len * batch_size, context)}
  }
  pub fn load_frames_f32(&mut self, frames: &[f32]) { self.out_act.borrow_mut().sync_load(frames); }
}

impl Operator for FrameInputOperator {
  fn batch_size(&self) -> usize { self.batch_cap }
  fn get_output_vars(&self) -> Option<SharedDeviceBuf<f32>> { Some(self.out_act.clone()) }
  fn forward(&mut self, _batch_size: usize, _phase: OpPhase) {}
  fn backward(&mut self, _batch_size: usize) {}
}

impl InputOperator for FrameInputOperator {
  fn downcast(&self) -> &Operator { self }
  fn expose_host_frame_buf(&mut self, batch_idx: usize) -> &mut [u8] {
    assert!(batch_idx < self.batch_cap);
    &mut self.in_buf_h[batch_idx * self.frame_len .. (batch_idx + 1) * self.frame_len]
  }
  /// `sync_load` of the staged frames, then the cast kernel (src/operator/mod.rs:640-664).
  fn load_frames(&mut self, batch_size: usize) {
    assert!(batch_size <= self.batch_cap);
    let n = batch_size * self.frame_len;
    self.in_buf.sync_load(&self.in_buf_h[ .. n]);
    let scale = if self.normalize { 1.0 / 255.0 } else { 1.0 };
    unwrap(unsafe { rh_cast_u8_f32(self.in_buf.as_ptr(), self.out_act.borrow_mut().as_mut_ptr(), n, scale,
                                   self.context.stream()) }, "rh_cast_u8_f32");
  }
  fn stage_shape(&mut self, _batch_idx: usize, _shape: (usize, usize, usize)) {}
}

pub enum OperatorConfig {
  Affine(AffineOperatorConfig),
  Conv2d(Conv2dOperatorConfig),
  Pool2d(Pool2dOperatorConfig),
}

pub struct SequentialOperatorWorker {
  batch_cap:   usize,
  shared_seed: [u64; 2],
  context:     Rc<DeviceContext>,
  input_op:    FrameInputOperator,
  hidden_ops:  Vec<Box<Operator>>,
  loss_op:     SoftmaxKLLossOperator,
}

impl SequentialOperatorWorker {
  pub fn new(batch_size: usize, capability: OpCapability, shared_seed: [u64; 2], in_frame_len: usize,
             hidden: &[OperatorConfig], loss: CategoricalLossConfig, context: Rc<DeviceContext>) -> SequentialOperatorWorker {
    let mut input_op = FrameInputOperator::new(batch_size, in_frame_len, false, context.clone());
    let mut hidden_ops: Vec<Box<Operator>> = Vec::with_capacity(hidden.len());
    for cfg in hidden.iter() {
      let op: Box<Operator> = {
        let prev: &mut Operator = match hidden_ops.last_mut() { Some(p) => &mut **p, None => &mut input_op };
        match *cfg {
          OperatorConfig::Affine(c) => Box::new(AffineOperator::new(batch_size, capability, c, prev, context.clone())),
          OperatorConfig::Conv2d(c) => Box::new(Conv2dOperator::new(batch_size, capability, c, prev, context.clone())),
          OperatorConfig::Pool2d(c) => Box::new(Pool2dOperator::new(batch_size, c, prev, context.clone())),
        }
      };
      hidden_ops.push(op);
    }
    let loss_op = SoftmaxKLLossOperator::new(batch_size, loss, &**hidden_ops.last().expect("a chain needs a hidden operator"),
                                             context);
    SequentialOperatorWorker{batch_cap: batch_size, shared_seed: shared_seed, context: context, input_op: input_op,
                             hidden_ops: hidden_ops, loss_op: loss_op}
  }
  pub fn frame_input_operator(&mut self) -> &mut FrameInputOperator { &mut self.input_op }

  /// `regularize -> accumulate_grads -> update_params -> reset` of every operator as ONE launch over the table of all
  /// parameter blocks (rh_sgd_momentum_step_multi): v = mu v + scale (g + l2 W); W += apply v; g = 0.  Same arithmetic
  /// per element as the four fan-outs of src/opt/sgd/new.rs:423-452.
  pub fn fused_sgd_step(&mut self, l2_reg_coef: f32, scale: f32, momentum: f32, apply: f32) {
    let mut rows: Vec<rh_sgd_tensor> = Vec::new();
    for op in self.hidden_ops.iter_mut() { op.sgd_tensors(l2_reg_coef, &mut rows); }
    if rows.is_empty() { return; }
    unwrap(unsafe { rh_sgd_momentum_step_multi(rows.len() as i32, rows.as_ptr(), scale, momentum, apply, 1,
                                               self.context.stream()) }, "rh_sgd_momentum_step_multi");
  }
}

fn write_file(path: &Path, blob: &[u8]) {
  let mut f = File::create(path).ok().expect("failed to create blob file");
  f.write_all(blob).ok().expect("failed to write blob file");
}

fn read_file(path: &Path) -> Vec<u8> {
  let mut blob = Vec::new();
  File::open(path).ok().expect("failed to open blob file").read_to_end(&mut blob).ok().expect("failed to read blob file");
  blob
}

impl Operator for SequentialOperatorWorker {
  fn batch_size(&self) -> usize { self.batch_cap }
  /// Every hidden operator gets two words of a xorshift128+ sequence seeded with the shared seed
  /// (src/operator/worker.rs:361-367), in chain order.
  fn init_params(&mut self, shared_seed: [u64; 2]) {
    let (mut s0, mut s1) = (shared_seed[0], shared_seed[1]);
    if s0 == 0 && s1 == 0 { s1 = 0x9E3779B97F4A7C15; }
    let mut next = move || {
      let mut x = s0;
      let y = s1;
      s0 = y;
      x ^= x << 23;
      s1 = x ^ y ^ (x >> 17) ^ (y >> 26);
      s1.wrapping_add(y)
    };
    for op in self.hidden_ops.iter_mut() {
      let a = next();
      let b = next();
      op.init_params([a, b]);
    }
  }
  fn forward(&mut self, batch_size: usize, phase: OpPhase) {
    self.input_op.forward(batch_size, phase);
    for op in self.hidden_ops.iter_mut() { op.forward(batch_size, phase); }
    self.loss_op.forward(batch_size, phase);
  }
  fn backward(&mut self, batch_size: usize) {
    self.loss_op.backward(batch_size);
    for op in self.hidden_ops.iter_mut().rev() { op.backward(batch_size); }
  }
  fn backward_scaled(&mut self, batch_size: usize, scale: f32) {
    self.loss_op.backward(batch_size);
    for op in self.hidden_ops.iter_mut().rev() { op.backward_scaled(batch_size, scale); }
  }
  fn regularize(&mut self, reg: Regularization) { for op in self.hidden_ops.iter_mut() { op.regularize(reg); } }
  fn accumulate_grads(&mut self, scale: f32, momentum: f32) {
    for op in self.hidden_ops.iter_mut() { op.accumulate_grads(scale, momentum); }
  }
  fn update_params(&mut self, scale: f32) { for op in self.hidden_ops.iter_mut() { op.update_params(scale); } }
  fn update_params2(&mut self, g: f32, u: f32) { for op in self.hidden_ops.iter_mut() { op.update_params2(g, u); } }
  fn save_params(&mut self) { for op in self.hidden_ops.iter_mut() { op.save_params(); } }
  fn restore_params(&mut self) { for op in self.hidden_ops.iter_mut() { op.restore_params(); } }
  fn reset(&mut self) { for op in self.hidden_ops.iter_mut() { op.reset(); } }
  fn descend(&mut self, scale: f32, l2: f32) { for op in self.hidden_ops.iter_mut() { op.descend(scale, l2); } }
  fn reset_gradients(&mut self, momentum: f32) { for op in self.hidden_ops.iter_mut() { op.reset_gradients(momentum); } }
  fn encode_params(&mut self, blob: &mut Vec<u8>) { for op in self.hidden_ops.iter_mut() { op.encode_params(blob); } }
  fn decode_params(&mut self, blob: &[u8]) -> usize {
    let mut off = 0;
    for op in self.hidden_ops.iter_mut() { off += op.decode_params(&blob[off ..]); }
    off
  }
  fn encode_state(&mut self, blob: &mut Vec<u8>) { for op in self.hidden_ops.iter_mut() { op.encode_state(blob); } }
  fn decode_state(&mut self, blob: &[u8]) -> usize {
    let mut off = 0;
    for op in self.hidden_ops.iter_mut() { off += op.decode_state(&blob[off ..]); }
    off
  }
}

impl OperatorWorker for SequentialOperatorWorker {
  fn num_workers(&self) -> usize { 1 }
  fn worker_rank(&self) -> usize { 0 }
  fn shared_seed(&self) -> [u64; 2] { self.shared_seed }
  fn input_operator(&mut self) -> &mut InputOperator { &mut self.input_op }
  fn loss_count(&self) -> usize { 1 }
  fn loss_operator(&mut self, rank: usize) -> &mut LossOperator {
    assert_eq!(rank, 0);
    &mut self.loss_op
  }
  /// `params.t_<t>.blob`, the `params.latest.blob` symlink, `checkpoint` (the iteration as a decimal line) with the
  /// previous one kept as `checkpoint.0` (src/operator/worker.rs:447-480).
  fn checkpoint_params(&mut self, t: usize, prefix: &Path) {
    fs::create_dir_all(prefix).ok();
    let mut blob = Vec::new();
    self.encode_params(&mut blob);
    let name = format!("params.t_{}.blob", t);
    write_file(&prefix.join(&name), &blob);
    let latest = prefix.join("params.latest.blob");
    fs::remove_file(&latest).ok();
    ::std::os::unix::fs::symlink(&PathBuf::from(&name), &latest).ok().expect("failed to symlink latest blob");
    let ck = prefix.join("checkpoint");
    if ck.exists() { fs::copy(&ck, &prefix.join("checkpoint.0")).ok(); }
    write_file(&ck, format!("{}\n", t).as_bytes());
  }
  fn checkpoint_state(&mut self, prefix: &Path) {
    fs::create_dir_all(prefix).ok();
    let mut blob = Vec::new();
    self.encode_state(&mut blob);
    write_file(&prefix.join(format!("state.latest.blob.{}", self.worker_rank())), &blob);
  }
  fn can_rollback(&mut self, prefix: &Path) -> Option<usize> {
    let mut text = String::new();
    match File::open(&prefix.join("checkpoint")) {
      Ok(mut f) => { f.read_to_string(&mut text).ok(); }
      Err(_) => return None,
    }
    text.lines().next().and_then(|l| l.trim().parse().ok())
  }
  fn rollback_params(&mut self, t: Option<usize>, prefix: &Path) {
    let path = match t {
      Some(t) => {
        let latest = self.can_rollback(prefix).expect("checkpoint file is missing or empty");
        assert!(t <= latest);
        prefix.join(format!("params.t_{}.blob", t))
      }
      None => prefix.join("params.latest.blob"),
    };
    let blob = read_file(&path);
    self.decode_params(&blob);
  }
  fn rollback_state(&mut self, prefix: &Path) {
    let blob = read_file(&prefix.join(format!("state.latest.blob.{}", self.worker_rank())));
    self.decode_state(&blob);
  }
}
