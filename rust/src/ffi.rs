//! Raw bindings of include/rembrandt_hip.h: the replacement for `rembrandt_kernels::ffi`,
//! `cuda_dnn::v4::ffi` and the cuBLAS/cudart calls of `array_cuda` on rembrandt's operator hot path.
//! Written for the reference's toolchain (rustc 1.9 nightly, `libc` crate); not compiled in the image
//! this library is built in (no Rust toolchain there).
#![allow(non_camel_case_types)]

use libc::{c_char, c_float, c_int, c_void, size_t};

pub type rh_stream_t = *mut c_void; // hipStream_t
pub enum rh_ctx {}
pub enum rh_graph {}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rh_conv_geom {
  pub n: i32, pub c: i32, pub h: i32, pub w: i32,
  pub k: i32, pub r: i32, pub s: i32,
  pub stride: i32, pub pad: i32,
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rh_pool_geom {
  pub n: i32, pub c: i32, pub h: i32, pub w: i32,
  pub size: i32, pub stride: i32, pub pad: i32,
  pub mode: i32,  // 0 max, 1 average (count includes padding)
  pub round: i32, // 0 floor (operator), 1 ceil (gen-1 layer)
}

#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rh_lrn_geom {
  pub n: i32, pub c: i32, pub h: i32, pub w: i32,
  pub size: i32,
  pub scale: c_float, pub power: c_float, pub min_div: c_float,
}

/// One parameter block of rh_sgd_momentum_step_multi (weights, gradient, momentum buffer).
#[repr(C)]
#[derive(Clone, Copy, Debug)]
pub struct rh_sgd_tensor {
  pub w: *mut f32,
  pub g: *mut f32,
  pub v: *mut f32,
  pub n: i64,
  pub l2: c_float,
  pub keep_grad: i32,  // nonzero: g is left as it is (the caller overwrites it, beta = 0, in its next backward pass)
}

pub const RH_CONV_FWD: c_int = 0;
pub const RH_CONV_BWD_FILTER: c_int = 1;
pub const RH_CONV_BWD_DATA: c_int = 2;
pub const RH_FUSE_BIAS: c_int = 0x10;
pub const RH_FUSE_RELU: c_int = 0x20;
pub const RH_MATH_BF16_MFMA_FP32ACC: c_int = 0x1;
pub const RH_ALGO_GATHER: c_int = 0x100;
pub const RH_ALGO_SCALAR_OFFSET: c_int = 0x200;
pub const RH_ALGO_WINOGRAD: c_int = 0x400;
pub const RH_ALGO_DIRECT: c_int = 0x800;
pub const RH_ALGO_SHARED_GPU: c_int = 0x1000;

#[link(name = "rembrandt_hip")]
extern "C" {
  pub fn rh_version() -> *const c_char;
  pub fn rh_error_string(code: c_int) -> *const c_char;
  pub fn rh_last_error() -> c_int;

  pub fn rh_ctx_create(device: c_int, out: *mut *mut rh_ctx) -> c_int;
  pub fn rh_ctx_destroy(ctx: *mut rh_ctx) -> c_int;
  pub fn rh_ctx_stream(ctx: *mut rh_ctx) -> rh_stream_t;
  pub fn rh_ctx_sync(ctx: *mut rh_ctx) -> c_int;
  pub fn rh_malloc(ctx: *mut rh_ctx, bytes: size_t, dptr: *mut *mut c_void) -> c_int;
  pub fn rh_free(ctx: *mut rh_ctx, dptr: *mut c_void) -> c_int;
  pub fn rh_load_overlapped(ctx: *mut rh_ctx, dst_d: *mut c_void, src_h: *const c_void, bytes: size_t) -> c_int;
  pub fn rh_mark_consumed(ctx: *mut rh_ctx) -> c_int;
  pub fn rh_store_begin(ctx: *mut rh_ctx, dst_h: *mut c_void, src_d: *const c_void, bytes: size_t) -> c_int;
  pub fn rh_store_wait(ctx: *mut rh_ctx) -> c_int;
  pub fn rh_host_malloc(ctx: *mut rh_ctx, bytes: size_t, hptr: *mut *mut c_void) -> c_int;
  pub fn rh_host_free(ctx: *mut rh_ctx, hptr: *mut c_void) -> c_int;
  pub fn rh_memset_f32(d: *mut f32, value: c_float, n: size_t, stream: rh_stream_t) -> c_int;
  pub fn rh_copy_d2d(dst: *mut c_void, src: *const c_void, bytes: size_t, stream: rh_stream_t) -> c_int;
  pub fn rh_load_sync(ctx: *mut rh_ctx, dst_d: *mut c_void, src_h: *const c_void, bytes: size_t) -> c_int;
  pub fn rh_store_sync(ctx: *mut rh_ctx, dst_h: *mut c_void, src_d: *const c_void, bytes: size_t) -> c_int;
  pub fn rh_cast_u8_f32(x: *const u8, y: *mut f32, n: size_t, scale: c_float, stream: rh_stream_t) -> c_int;

  pub fn rh_conv2d_out_dim(input: i32, size: i32, stride: i32, pad: i32) -> i32;
  pub fn rh_pool2d_out_dim(input: i32, size: i32, stride: i32, pad: i32, round: i32) -> i32;
  pub fn rh_conv2d_winograd_flops(g: *const rh_conv_geom, pass: c_int, flags: c_int) -> f64;
  pub fn rh_conv2d_workspace_bytes(g: *const rh_conv_geom, pass: c_int) -> size_t;
  pub fn rh_conv2d_workspace_bytes_upto(g: *const rh_conv_geom, pass: c_int) -> size_t;
  pub fn rh_conv2d_fwd(g: *const rh_conv_geom, alpha: c_float, x: *const f32, w: *const f32, beta: c_float,
                       y: *mut f32, bias: *const f32, ws: *mut c_void, ws_bytes: size_t, flags: c_int,
                       stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_bwd_filter(g: *const rh_conv_geom, alpha: c_float, x: *const f32, dy: *const f32,
                              beta: c_float, dw: *mut f32, ws: *mut c_void, ws_bytes: size_t, flags: c_int,
                              stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_bwd_bias(n: i32, k: i32, plane: i32, alpha: c_float, dy: *const f32, beta: c_float,
                            db: *mut f32, stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_bwd_bias_workspace_bytes(n: i32, k: i32, plane: i32) -> size_t;
  pub fn rh_conv2d_bwd_bias_ws(n: i32, k: i32, plane: i32, alpha: c_float, dy: *const f32, beta: c_float,
                               db: *mut f32, ws: *mut c_void, ws_bytes: size_t, stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_bwd_data(g: *const rh_conv_geom, alpha: c_float, w: *const f32, dy: *const f32,
                            beta: c_float, dx: *mut f32, ws: *mut c_void, ws_bytes: size_t, flags: c_int,
                            stream: rh_stream_t) -> c_int;
  // Filter and bias gradient in one call: dy is read once where the filter gradient copies it anyway.
  pub fn rh_conv2d_bwd_filter_bias(g: *const rh_conv_geom, alpha: c_float, x: *const f32, dy: *const f32,
                                   beta: c_float, dw: *mut f32, db: *mut f32, ws: *mut c_void, ws_bytes: size_t,
                                   flags: c_int, stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_bwd_bias_workspace_bytes_upto(n: i32, k: i32, plane: i32) -> size_t;
  // The two-stage bias gradient on the library's own static scratch (callers that cannot allocate).
  pub fn rh_noalloc_scratch_bytes() -> size_t;
  pub fn rh_conv2d_bwd_bias_noalloc(n: i32, k: i32, plane: i32, alpha: c_float, dy: *const f32, beta: c_float,
                                    db: *mut f32, stream: rh_stream_t) -> c_int;
  // Data gradient that also applies the backward mask of the ReLU that produced this layer's input (x_act).
  pub fn rh_conv2d_bwd_data_relu_supported(g: *const rh_conv_geom) -> c_int;
  pub fn rh_conv2d_bwd_data_relu(g: *const rh_conv_geom, alpha: c_float, w: *const f32, dy: *const f32,
                                 beta: c_float, dx: *mut f32, x_act: *const f32, ws: *mut c_void, ws_bytes: size_t,
                                 flags: c_int, stream: rh_stream_t) -> c_int;

  pub fn rh_add_bias_nchw(bias: *const f32, y: *mut f32, plane: i32, k: i32, n: i32, alpha: c_float,
                          beta: c_float, stream: rh_stream_t) -> c_int;
  // Same names and argument lists as rembrandt_kernels::ffi (src/operator/mod.rs:1108-1113, 1154-1160).
  pub fn rembrandt_kernel_batch_map_rect_inplace(y: *mut f32, frame_len: i32, batch: i32, stream: rh_stream_t);
  pub fn rembrandt_kernel_batch_map_rect_backprop_inplace(y: *const f32, frame_len: i32, batch: i32,
                                                          dy: *mut f32, stream: rh_stream_t);

  pub fn rh_sgemm_workspace_bytes(m: i32, n: i32, k: i32) -> size_t;
  pub fn rh_sgemm(trans_a: c_int, trans_b: c_int, m: i32, n: i32, k: i32, alpha: c_float, a: *const f32,
                  lda: i32, b: *const f32, ldb: i32, beta: c_float, c: *mut f32, ldc: i32, ws: *mut c_void,
                  ws_bytes: size_t, flags: c_int, stream: rh_stream_t) -> c_int;
  pub fn rh_sgemm_workspace_bytes_upto(m: i32, n: i32, k: i32, which: c_int) -> size_t;
  pub fn rh_sgemm_bias_act(trans_a: c_int, trans_b: c_int, m: i32, n: i32, k: i32, alpha: c_float, a: *const f32,
                           lda: i32, b: *const f32, ldb: i32, beta: c_float, c: *mut f32, ldc: i32, bias: *const f32,
                           ws: *mut c_void, ws_bytes: size_t, flags: c_int, stream: rh_stream_t) -> c_int;
  pub fn rh_saxpy(n: i64, alpha: c_float, x: *const f32, y: *mut f32, stream: rh_stream_t) -> c_int;
  pub fn rh_sscal(n: i64, alpha: c_float, x: *mut f32, stream: rh_stream_t) -> c_int;

  pub fn rh_pool2d_fwd(g: *const rh_pool_geom, x: *const f32, y: *mut f32, opt_argmax: *mut i32,
                       stream: rh_stream_t) -> c_int;
  pub fn rh_pool2d_bwd(g: *const rh_pool_geom, x: *const f32, y: *const f32, dy: *const f32, dx: *mut f32,
                       opt_argmax: *const i32, stream: rh_stream_t) -> c_int;

  // Max pooling with a one-byte mask (the winner's slot inside its window) for an operator's private use.
  pub fn rh_pool2d_slot_supported(g: *const rh_pool_geom) -> c_int;
  pub fn rh_pool2d_fwd_slot(g: *const rh_pool_geom, x: *const f32, y: *mut f32, slot: *mut u8, stream: rh_stream_t) -> c_int;
  pub fn rh_pool2d_bwd_slot(g: *const rh_pool_geom, relu_y: *const f32, dy: *const f32, dx: *mut f32, slot: *const u8,
                            stream: rh_stream_t) -> c_int;

  pub fn rh_softmax_fwd(x: *const f32, p: *mut f32, c: i32, n: i32, stream: rh_stream_t) -> c_int;
  // Same names and argument lists as rembrandt_kernels::ffi (src/operator/loss.rs:132-140, 191-210, 229-239).
  pub fn rembrandt_kernel_batch_map_softmax_kl_backward(p: *const f32, c: i32, n: i32, labels: *const i32,
                                                        weights: *const f32, dx: *mut f32, stream: rh_stream_t);
  pub fn rembrandt_kernel_batch_map_softmax_kl_loss1(p: *const f32, c: i32, n: i32, labels: *const i32,
                                                     weights: *const f32, beta: c_float, loss1: *mut f32,
                                                     stream: rh_stream_t);
  pub fn rembrandt_kernel_batch_blockreduce_sum(src: *const f32, len: i32, batch: i32, dst: *mut f32,
                                                beta: c_float, stream: rh_stream_t);
  pub fn rembrandt_kernel_batch_blockreduce_argmax(src: *const f32, len: i32, batch: i32, max_out: *mut f32,
                                                   idx_out: *mut i32, stream: rh_stream_t);

  // The five loss-operator calls of a train step as one launch (bit-identical to them).
  pub fn rh_softmax_kl_step(x: *const f32, c: i32, n: i32, labels: *const i32, weights: *const f32, p: *mut f32,
                            max_out: *mut f32, idx_out: *mut i32, loss1: *mut f32, loss_sum: *mut f32, dx: *mut f32,
                            counter: *mut u32, stream: rh_stream_t) -> c_int;
  // The classifier tail of a train step (two affine layers, the loss step, their data gradients) and its parameter
  // gradients, one launch each.
  pub fn rh_affine2_softmax_kl_step_supported(b: i32, i: i32, h: i32, c: i32) -> c_int;
  pub fn rh_affine2_softmax_kl_step(b: i32, i: i32, h: i32, c: i32, relu1: i32, x: *const f32, w1: *const f32, b1: *const f32,
                                    w2: *const f32, b2: *const f32, labels: *const i32, weights: *const f32, h_out: *mut f32,
                                    logits: *mut f32, p: *mut f32, max_out: *mut f32, idx_out: *mut i32, loss1: *mut f32,
                                    loss_sum: *mut f32, dlogits: *mut f32, dh: *mut f32, dx: *mut f32, counter: *mut u32,
                                    stream: rh_stream_t) -> c_int;
  pub fn rh_affine2_bwd_params(b: i32, i: i32, h: i32, c: i32, x: *const f32, h_act: *const f32, dh: *const f32,
                               dlogits: *const f32, beta1: c_float, dw1: *mut f32, db1: *mut f32, beta2: c_float,
                               dw2: *mut f32, db2: *mut f32, stream: rh_stream_t) -> c_int;
  // Host generator behind init_params (the reference's random stream lives in crates outside its tree).
  pub fn rh_rng_fill_uniform(seed: u64, stream_id: u64, host: *mut f32, n: size_t, lo: c_float, hi: c_float) -> c_int;
  pub fn rh_rng_fill_normal(seed: u64, stream_id: u64, host: *mut f32, n: size_t, mean: c_float, std: c_float) -> c_int;
  pub fn rh_rng_fill_int(seed: u64, stream_id: u64, host: *mut i32, n: size_t, modulus: i32) -> c_int;

  pub fn rh_sgd_momentum_step(n: i64, w: *mut f32, g: *mut f32, v: *mut f32, l2: c_float, scale: c_float,
                              mu: c_float, apply: c_float, zero_grad: c_int, stream: rh_stream_t) -> c_int;
  // One launch over a table of parameter blocks: what one `update` fan-out over a chain of operators issues.
  pub fn rh_sgd_momentum_step_multi(count: i32, tensors: *const rh_sgd_tensor, scale: c_float, mu: c_float,
                                    apply: c_float, zero_grad: c_int, stream: rh_stream_t) -> c_int;
  pub fn rh_descend(n: i64, w: *mut f32, g: *mut f32, s: c_float, l2: c_float, stream: rh_stream_t) -> c_int;

  // Second stream of the context (no counterpart in the reference, which issues everything on ctx.stream).
  pub fn rh_ctx_aux_stream(ctx: *mut rh_ctx) -> rh_stream_t;
  pub fn rh_ctx_fork(ctx: *mut rh_ctx) -> c_int;
  pub fn rh_ctx_join(ctx: *mut rh_ctx) -> c_int;

  // Stream capture: launches between begin and end are recorded into a HIP graph; rh_graph_launch replays them.
  pub fn rh_ctx_begin_capture(ctx: *mut rh_ctx) -> c_int;
  pub fn rh_ctx_end_capture(ctx: *mut rh_ctx, out: *mut *mut rh_graph) -> c_int;
  pub fn rh_graph_launch(g: *mut rh_graph, ctx: *mut rh_ctx) -> c_int;
  pub fn rh_graph_destroy(g: *mut rh_graph) -> c_int;

  // Max-pool backward that also applies the ReLU backward mask of the operator below (one pass instead of two).
  pub fn rh_pool2d_bwd_relu_supported(g: *const rh_pool_geom) -> c_int;
  pub fn rh_pool2d_bwd_relu(g: *const rh_pool_geom, y: *const f32, dy: *const f32, dx: *mut f32,
                            argmax: *const i32, stream: rh_stream_t) -> c_int;
  pub fn rh_pool2d_bwd_avg_relu(g: *const rh_pool_geom, x: *const f32, dy: *const f32, dx: *mut f32, stream: rh_stream_t) -> c_int;

  // Data3dOperator preprocessing (src/operator/mod.rs:666-691, 716-725, 767-773) and dropout (mod.rs:2220-2246).
  pub fn rh_crop_nchw(src: *const f32, dst: *mut f32, planes: i64, in_w: i32, in_h: i32, crop_w: i32, crop_h: i32,
                      off_w: i32, off_h: i32, stream: rh_stream_t) -> c_int;
  pub fn rembrandt_kernel_batch_blockmap256_flip(src: *const f32, width: i32, rows: i32, dst: *mut f32,
                                                 stream: rh_stream_t);
  pub fn rembrandt_kernel_batch_map_preproc_pca3_noise(src: *const f32, spatial: i32, batch: i32,
                                                       alphas: *const f32, svals: *const f32, svecs: *const f32,
                                                       dst: *mut f32, stream: rh_stream_t);
  pub fn rembrandt_kernel_map_dropout(input: *const f32, n: i32, drop_ratio: c_float, scale: c_float,
                                      rnd: *const f32, out: *mut f32, mask: *mut i32, stream: rh_stream_t);
  pub fn rembrandt_kernel_map_dropout_backprop(out_delta: *const f32, n: i32, drop_ratio: c_float, scale: c_float,
                                               mask: *const i32, in_delta: *mut f32, stream: rh_stream_t);
  pub fn rh_rng_fill_uniform01_device(seed: u64, stream_id: u64, first: u64, dst: *mut f32, n: size_t,
                                      stream: rh_stream_t) -> c_int;
  pub fn rh_lrn_fwd(g: *const rh_lrn_geom, x: *const f32, y: *mut f32, denom: *mut f32, stream: rh_stream_t) -> c_int;
  pub fn rh_lrn_bwd(g: *const rh_lrn_geom, x: *const f32, y: *const f32, denom: *const f32, dy: *const f32,
                    dx: *mut f32, stream: rh_stream_t) -> c_int;

  // CudnnBatchNormOp in Spatial mode (src/operator/conv.rs:493-535, 594-607): same alpha/beta pairs and buffer order.
  pub fn rh_bnorm_workspace_bytes(n: c_int, c: c_int, plane: c_int) -> size_t;
  pub fn rh_bnorm_workspace_bytes_upto(n: c_int, c: c_int, plane: c_int) -> size_t;
  pub fn rh_bnorm_fwd_train(n: c_int, c: c_int, plane: c_int, alpha: c_float, x: *const f32, beta: c_float,
                            y: *mut f32, ema_factor: f64, epsilon: f64, scale: *const f32, bias: *const f32,
                            running_mean: *mut f32, running_ivar: *mut f32, cached_mean: *mut f32,
                            cached_ivar: *mut f32, ws: *mut c_void, ws_bytes: size_t, flags: c_int,
                            stream: rh_stream_t) -> c_int;
  pub fn rh_bnorm_fwd_infer(n: c_int, c: c_int, plane: c_int, alpha: c_float, x: *const f32, beta: c_float,
                            y: *mut f32, epsilon: f64, scale: *const f32, bias: *const f32,
                            running_mean: *const f32, running_ivar: *const f32, ws: *mut c_void, ws_bytes: size_t,
                            flags: c_int, stream: rh_stream_t) -> c_int;
  pub fn rh_bnorm_bwd(n: c_int, c: c_int, plane: c_int, alpha_data: c_float, beta_data: c_float, x: *const f32,
                      dy: *const f32, dx: *mut f32, alpha_param: c_float, beta_param: c_float, epsilon: f64,
                      scale: *const f32, dscale: *mut f32, dbias: *mut f32, cached_mean: *const f32,
                      cached_ivar: *const f32, ws: *mut c_void, ws_bytes: size_t, stream: rh_stream_t) -> c_int;
  pub fn rh_bnorm_bwd_relu(n: c_int, c: c_int, plane: c_int, alpha_data: c_float, beta_data: c_float, x: *const f32,
                           dy: *const f32, dx: *mut f32, alpha_param: c_float, beta_param: c_float, epsilon: f64,
                           scale: *const f32, bias: *const f32, dscale: *mut f32, dbias: *mut f32,
                           cached_mean: *const f32, cached_ivar: *const f32, ws: *mut c_void, ws_bytes: size_t,
                           stream: rh_stream_t) -> c_int;

  // Packed bf16 activations for forward-only chains: producers write the consumer's operand, filters are converted once.
  pub fn rh_bf16_act_bytes(n: i32, c: i32, h: i32, w: i32, halo: i32) -> size_t;
  pub fn rh_bf16_pack_nchw(n: i32, c: i32, h: i32, w: i32, halo: i32, x: *const f32, xp: *mut c_void,
                           stream: rh_stream_t) -> c_int;
  pub fn rh_bf16_unpack_nchw(n: i32, c: i32, h: i32, w: i32, halo: i32, xp: *const c_void, x: *mut f32,
                             stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_fwd_bf16_filter_bytes(g: *const rh_conv_geom) -> size_t;
  pub fn rh_conv2d_fwd_bf16_takes_packed(g: *const rh_conv_geom) -> c_int;
  pub fn rh_conv2d_fwd_bf16_workspace_bytes(g: *const rh_conv_geom) -> size_t;
  pub fn rh_conv2d_fwd_bf16_prep_filter(g: *const rh_conv_geom, w: *const f32, wprep: *mut c_void, wprep_bytes: size_t,
                                        stream: rh_stream_t) -> c_int;
  pub fn rh_conv2d_fwd_bf16_packed(g: *const rh_conv_geom, xp: *const c_void, x: *const f32, wprep: *const c_void,
                                   bias: *const f32, y: *mut f32, yp: *mut c_void, yp_halo: i32, ws: *mut c_void,
                                   ws_bytes: size_t, flags: c_int, stream: rh_stream_t) -> c_int;
  pub fn rh_pool2d_fwd_bf16_packed(g: *const rh_pool_geom, xp: *const c_void, yp: *mut c_void, yp_halo: i32,
                                   stream: rh_stream_t) -> c_int;

  // Per-launch timing and the calibration launches of the roofline report (no counterpart in the reference).
  pub fn rh_profile_enable(on: c_int) -> c_int;
  pub fn rh_profile_enabled() -> c_int;
  pub fn rh_profile_filter(prefix: *const c_char) -> c_int;
  pub fn rh_profile_count() -> c_int;
  pub fn rh_profile_get(i: c_int, tag: *mut *const c_char, work: *mut f64, ms: *mut c_float) -> c_int;
  pub fn rh_profile_reset() -> c_int;
  pub fn rh_probe_mfma_loop(blocks: c_int, nacc: c_int, iters: c_int, sink: *mut f32, stream: rh_stream_t) -> c_int;
  pub fn rh_probe_mfma_loop_varied(blocks: c_int, iters: c_int, sink: *mut f32, stream: rh_stream_t) -> c_int;
  pub fn rh_probe_copy(src: *const f32, dst: *mut f32, n: size_t, stream: rh_stream_t) -> c_int;
}

/// The reference `unwrap()`s / `panic!`s on every native error (src/operator/mod.rs:1685-1696).
pub fn unwrap(code: c_int, what: &str) {
  if code != 0 {
    let msg = unsafe { ::std::ffi::CStr::from_ptr(rh_error_string(code)) };
    panic!("{} failed: {} ({:?})", what, code, msg);
  }
}
