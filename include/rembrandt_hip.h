/*
 * rembrandt_hip.h -- C ABI of librembrandt_hip.so: the MI355X (gfx950) replacement for the native
 * layer underneath rembrandt's single-GPU operator hot path.
 *
 * In the reference that native layer is three crates whose sources are not in its tree:
 * `cuda_dnn::v4` (cuDNN), `array_cuda` (cuBLAS + device memory / streams) and
 * `rembrandt_kernels::ffi` (hand-written kernels).  Each entry point below names the reference
 * call site(s) it replaces (paths relative to the reference tree).
 *
 * Conventions
 *   - plain pointers and sizes only; device pointers unless a parameter is named `*_h` / `host`;
 *   - every `rh_*` function returns 0 on success, a positive hipError_t value on a HIP failure,
 *     or a negative RH_E_* code on a usage error.  The reference panics on every error
 *     (`.unwrap()` / `panic!`, src/operator/mod.rs:1685-1696); a binding reproduces that by
 *     unwrapping the return code.  The `rembrandt_kernel_*` symbols keep the reference's
 *     `void` signatures; their launch status can be read with rh_last_error();
 *   - nothing here allocates, frees or synchronises unless its name says so (`rh_malloc`,
 *     `rh_free`, `*_sync`); all work is enqueued on the given stream;
 *   - tensors are fp32, NCHW with W fastest (src/operator/mod.rs:1471-1474); filters
 *     [K][C][R][S]; 2-D arrays are column-major with the first index fastest
 *     (src/arch_new.rs:141-145), so an affine weight `(in, out)` is `[out][in]` in memory;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 */
#ifndef REMBRANDT_HIP_H
#define REMBRANDT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* rh_stream_t; /* hipStream_t */

/* usage errors */
#define RH_E_INVALID   (-1) /* bad argument (NULL pointer, non-positive dimension, unknown enum) */
#define RH_E_WORKSPACE (-2) /* workspace missing or smaller than rh_conv2d_workspace_bytes()      */
#define RH_E_UNSUPPORTED (-3)
#define RH_E_LIMIT     (-4) /* size beyond a documented limit                                      */

/* math / fusion flags of the conv and GEMM entry points */
#define RH_MATH_FP32_MFMA          0x0  /* fp32 operands, v_mfma_f32_32x32x2_f32, fp32 accumulate (default) */
#define RH_MATH_BF16_MFMA_FP32ACC  0x1  /* operands rounded to bf16 (RNE) on load, bf16 MFMA, fp32 accumulate */
#define RH_FUSE_BIAS               0x10 /* conv fwd: add bias[k] in the epilogue (replaces the separate K2 pass) */
#define RH_FUSE_RELU               0x20 /* conv fwd: max(.,0) in the epilogue (replaces the separate K3 pass)    */
/* loader family of the conv passes; neither bit = the library chooses (what the operators use) */
#define RH_ALGO_GATHER             0x100 /* k -> {offset, dr, ds} table gather straight from the NCHW tensors      */
#define RH_ALGO_SCALAR_OFFSET      0x200 /* scalar-offset loads on padded / transposed copies in the workspace,
                                            wherever the geometry allows it (else the gather family)             */
#define RH_ALGO_WINOGRAD           0x400 /* every pass of a 3x3 stride-1 layer by Winograd F(2x2, 3x3): 2.25x
                                            fewer multiply-adds, sums in another order; the forward pass of a 5x5
                                            stride-1 layer in the same form (its filter as four 3x3 blocks: 1.56x
                                            fewer).  RH_E_UNSUPPORTED for other geometries and passes.  Without an
                                            RH_ALGO_* bit the library takes it for such layers of 64 channels and more
                                            on both sides; either bit above keeps the direct form */
#define RH_ALGO_DIRECT             0x800 /* never the Winograd form; the direct forms chosen as without any RH_ALGO_* bit */
#define RH_ALGO_SHARED_GPU         0x1000 /* a hint, with any of the above: kernels of another stream run beside this call.
                                             Forms that spend compute-unit time to shorten the call's own last round of
                                             blocks (the Winograd kernels' sliced tail blocks) are not taken: beside
                                             other work the idle units of that round are not idle (measured: the
                                             ResNet-18 template step 26.5 -> 26.1 ms).  Same result up to summation order. */

const char* rh_version(void);
/* Status of the most recent launch made by a void `rembrandt_kernel_*` entry point on this thread. */
int rh_last_error(void);
const char* rh_error_string(int code);

/* ---------------------------------------------------------------------------------------------
 * Context + memory.  Replaces array_cuda::device::{context,memory}: DeviceContext::new(dev)
 * (tools/train-mnist.rs:155-178), ctx.stream.ptr (src/operator/mod.rs:1112), ctx.sync()
 * (src/operator/comm.rs:223), DeviceBuffer::zeros (mod.rs:940), send (mod.rs:1249-1267),
 * sync_load / sync_store (src/operator/loss.rs:170-186, 212-213), set_constant (mod.rs:908-909),
 * cast_bytes{,_normalized} (mod.rs:735-737).
 * ------------------------------------------------------------------------------------------- */
typedef struct rh_ctx rh_ctx;
int rh_ctx_create(int device, rh_ctx** out);
int rh_ctx_destroy(rh_ctx* ctx);
rh_stream_t rh_ctx_stream(rh_ctx* ctx);
int rh_ctx_sync(rh_ctx* ctx);                       /* every stream of the context */
/* A second stream of the context (default priority, created on first use) for launches that may overlap the main
 * stream's, e.g. a layer's filter gradient beside its data gradient.  rh_ctx_fork: the second stream waits for what
 * the main stream holds now; rh_ctx_join: the main stream waits for what the second holds now.  No host blocking. */
rh_stream_t rh_ctx_aux_stream(rh_ctx* ctx);
int rh_ctx_fork(rh_ctx* ctx);
int rh_ctx_join(rh_ctx* ctx);
/* Stream capture (no counterpart in the reference, which launches every kernel of every step from the host): between
 * rh_ctx_begin_capture and rh_ctx_end_capture the launches made on the context's streams are recorded into a HIP graph
 * instead of executed; rh_graph_launch replays the recording on the main stream.  For launch-bound sequences (a whole
 * train step of a LeNet-sized network is ~60 launches of a few microseconds).  Only kernel launches and
 * device-to-device copies may be recorded: calls that copy to or from the host, synchronise, allocate or memset return
 * an error or break the recording.  rh_ctx_end_capture(ctx, NULL) discards a recording. */
typedef struct rh_graph rh_graph;
int rh_ctx_begin_capture(rh_ctx* ctx);
int rh_ctx_end_capture(rh_ctx* ctx, rh_graph** out);
int rh_graph_launch(rh_graph* g, rh_ctx* ctx);
int rh_graph_destroy(rh_graph* g);
int rh_malloc(rh_ctx* ctx, size_t bytes, void** dptr); /* zero-filled, like DeviceBuffer::zeros */
int rh_free(rh_ctx* ctx, void* dptr);
/* Page-locked, zero-filled host memory for what is copied to the device every batch: the u8 frame buffer that
 * Data3dOperator stages its input in (in_buf_h, src/operator/mod.rs:640-700; a plain Vec<u8> there). */
int rh_host_malloc(rh_ctx* ctx, size_t bytes, void** hptr);
int rh_host_free(rh_ctx* ctx, void* hptr);
int rh_memset_f32(float* d, float value, size_t n, rh_stream_t stream);
int rh_copy_d2d(void* dst, const void* src, size_t bytes, rh_stream_t stream);
int rh_load_sync(rh_ctx* ctx, void* dst_d, const void* src_h, size_t bytes);
int rh_store_sync(rh_ctx* ctx, void* dst_h, const void* src_d, size_t bytes);
/* sync_load of the per-batch input (Data3dOperator::load_frames, src/operator/mod.rs:690-700) without the wait for
 * the kernels still queued on the context's stream: the copy runs on a stream of its own, after the last reader of
 * dst_d that rh_mark_consumed recorded, and later work on the context's stream waits for it.  Returns when src_h may
 * be reused.  Falls back to waiting for the context's stream when no reader was marked (first load, or the readers
 * ran inside a recorded graph); RH_E_UNSUPPORTED between rh_ctx_begin_capture and rh_ctx_end_capture. */
int rh_load_overlapped(rh_ctx* ctx, void* dst_d, const void* src_h, size_t bytes);
int rh_mark_consumed(rh_ctx* ctx);
/* sync_store of the per-batch results (the predicted categories and the loss, src/operator/loss.rs:170-186, 212-213)
 * in two halves, so that the host's wait does not have to come before the backward pass is enqueued: rh_store_begin
 * copies src_d to dst_h on the copy stream as soon as what the context's stream holds now is complete, without
 * delaying launches made after the call; rh_store_wait blocks until every copy begun so far has landed.  dst_h is
 * page-locked memory from rh_host_malloc; launches enqueued between the two calls must not write src_d.
 * RH_E_UNSUPPORTED between rh_ctx_begin_capture and rh_ctx_end_capture. */
int rh_store_begin(rh_ctx* ctx, void* dst_h, const void* src_d, size_t bytes);
int rh_store_wait(rh_ctx* ctx);
int rh_cast_u8_f32(const uint8_t* x, float* y, size_t n, float scale, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Convolution.  Replaces cuda_dnn::v4 CudnnConvFwdOp::forward (src/operator/mod.rs:1684-1696,
 * src/layer_new.rs:999-1011, src/layer.rs:1414-1420), CudnnConvBwdFilterOp::backward_filter
 * (mod.rs:1765-1774, layer_new.rs:1092-1101), ::backward_bias (mod.rs:1775-1781) and
 * CudnnConvBwdDataOp::backward_data (mod.rs:1783-1793).  Cross-correlation, symmetric padding,
 * square stride; output extent max(0, in + 2*pad - size + stride) / stride (mod.rs:1393-1398).
 * ------------------------------------------------------------------------------------------- */
typedef struct {
  int32_t N, C, H, W; /* input  N x C x H x W */
  int32_t K, R, S;    /* filter K x C x R x S */
  int32_t stride, pad;
} rh_conv_geom;

enum { RH_CONV_FWD = 0, RH_CONV_BWD_FILTER = 1, RH_CONV_BWD_DATA = 2 };

int32_t rh_conv2d_out_dim(int32_t in, int32_t size, int32_t stride, int32_t pad);
/* Bytes of scratch the given pass needs whatever flags it is called with (0 is possible).  The scratch must be
 * 256-byte aligned. */
size_t rh_conv2d_workspace_bytes(const rh_conv_geom* g, int pass);
/* The same for a scratch buffer that is allocated once and then used with every batch 1..g->N, the way the
 * reference's operators size theirs for batch_cap (src/operator/mod.rs:1493-1507): the largest need of any such
 * batch.  The need is not monotone in N (a pass with few result tiles cuts its contraction into slices and keeps
 * their partial sums in the scratch), so this can exceed rh_conv2d_workspace_bytes of g itself. */
size_t rh_conv2d_workspace_bytes_upto(const rh_conv_geom* g, int pass);
/* FLOPs (2 per multiply-add) that a pass (RH_CONV_FWD, RH_CONV_BWD_DATA, RH_CONV_BWD_FILTER) executes on this geometry when the library takes
 * the Winograd F(2x2, 3x3) form for it under `flags` (16 multiply-adds per 2x2 output tile, filter and channel; tiles
 * that hang over an odd extent count whole), 0 when it takes a direct form.  The direct form's count is
 * 2 * N*K*P*Q * C*R*S.  No counterpart in the reference (cuDNN picks its algorithm through cudnnGet*Algorithm,
 * src/operator/mod.rs:1629-1661, and never says what it costs). */
double rh_conv2d_winograd_flops(const rh_conv_geom* g, int pass, int flags);

/* y = alpha * corr(x, w) + beta * y.  With RH_FUSE_BIAS, `bias` (length K) is added after the
 * alpha/beta blend; with RH_FUSE_RELU the result is clamped at 0.  bias may be NULL otherwise. */
int rh_conv2d_fwd(const rh_conv_geom* g, float alpha, const float* x, const float* w, float beta,
                  float* y, const float* bias, void* ws, size_t ws_bytes, int flags,
                  rh_stream_t stream);
/* dw = alpha * sum_{n,p,q} dy * x + beta * dw.  Deterministic two-pass split reduction. */
int rh_conv2d_bwd_filter(const rh_conv_geom* g, float alpha, const float* x, const float* dy,
                         float beta, float* dw, void* ws, size_t ws_bytes, int flags,
                         rh_stream_t stream);
/* rh_conv2d_bwd_filter followed by rh_conv2d_bwd_bias (mod.rs:1765-1781) with the same alpha and beta, as one call:
 * db = alpha * sum_{n,p,q} dy + beta * db as well.  Where the filter gradient makes a pass of its own over dy (the
 * channel-last copy of the large layers) that pass also leaves the plane sums, so dy is not read a second time.
 * Scratch as for rh_conv2d_bwd_filter (rh_conv2d_workspace_bytes covers both). */
int rh_conv2d_bwd_filter_bias(const rh_conv_geom* g, float alpha, const float* x, const float* dy, float beta,
                              float* dw, float* db, void* ws, size_t ws_bytes, int flags, rh_stream_t stream);
/* db[k] = alpha * sum_{n,p,q} dy[n,k,p,q] + beta * db[k];  plane = P*Q. */
int rh_conv2d_bwd_bias(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy,
                       float beta, float* db, rh_stream_t stream);
/* Same result through a two-stage reduction that fills the GPU when K is small (scratch from the caller;
 * without scratch it falls back to the one-stage form). */
size_t rh_conv2d_bwd_bias_workspace_bytes(int32_t N, int32_t K, int32_t plane);
size_t rh_conv2d_bwd_bias_workspace_bytes_upto(int32_t N, int32_t K, int32_t plane); /* largest need of N' = 1..N */
int rh_conv2d_bwd_bias_ws(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy, float beta,
                          float* db, void* ws, size_t ws_bytes, rh_stream_t stream);
/* rh_conv2d_bwd_bias_ws without the scratch argument and without any allocation.  It has no counterpart in the
 * reference; it is for callers that cannot allocate device memory or hand over a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The scratch of the two-stage reduction lives in an
 * 8 MiB device array inside the library (rh_noalloc_scratch_bytes(); every GPU the library is used on holds its own
 * copy until the process ends), whose address is looked up once per device by rh_ctx_create, or by the first call on
 * a device with that device current.  Geometries whose scratch need (rh_conv2d_bwd_bias_workspace_bytes) exceeds the
 * array return RH_E_LIMIT.  All calls on one GPU share the array: calls that overlap in time on one GPU (different
 * streams, different threads) race; order them.  Nothing in the array has to be cleared between calls. */
size_t rh_noalloc_scratch_bytes(void);
int rh_conv2d_bwd_bias_noalloc(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy, float beta,
                               float* db, rh_stream_t stream);
/* dx = alpha * corr^T(dy, w) + beta * dx. */
int rh_conv2d_bwd_data(const rh_conv_geom* g, float alpha, const float* w, const float* dy,
                       float beta, float* dx, void* ws, size_t ws_bytes, int flags,
                       rh_stream_t stream);
/* rh_conv2d_bwd_data followed by the in-place ReLU backward of the operator below (the
 * rembrandt_kernel_batch_map_rect_backprop_inplace(x_act, ., ., dx) that opens that operator's backward, mod.rs:1730-1737),
 * as one call: dx[i] = x_act[i] > 0 ? alpha * corr^T(dy, w)[i] + beta * dx[i] : 0, where x_act is this convolution's
 * input, i.e. that ReLU's output.  Same values as the two calls, without the extra pass over dx.
 * rh_conv2d_bwd_data_relu_supported: nonzero for the geometries that have this form (all with stride 1). */
int rh_conv2d_bwd_data_relu_supported(const rh_conv_geom* g);
int rh_conv2d_bwd_data_relu(const rh_conv_geom* g, float alpha, const float* w, const float* dy, float beta,
                            float* dx, const float* x_act, void* ws, size_t ws_bytes, int flags, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Bias add and ReLU.  rh_add_bias_nchw replaces CudnnAddOp::forward (mod.rs:1097-1103,
 * 1697-1704): y[n,k,:] = alpha*bias[k] + beta*y[n,k,:].  The two rembrandt_kernel_* symbols keep
 * the names and argument lists of rembrandt_kernels::ffi as seen at mod.rs:1108-1113,
 * 1154-1160, 1709-1714, 1754-1760 (the stream argument is a hipStream_t).
 * ------------------------------------------------------------------------------------------- */
int rh_add_bias_nchw(const float* bias, float* y, int32_t plane, int32_t K, int32_t N, float alpha,
                     float beta, rh_stream_t stream);
void rembrandt_kernel_batch_map_rect_inplace(float* y, int32_t frame_len, int32_t batch,
                                             rh_stream_t stream);
void rembrandt_kernel_batch_map_rect_backprop_inplace(const float* y, int32_t frame_len,
                                                      int32_t batch, float* dy, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Column-major SGEMM and BLAS-1.  Replaces array_cuda's BlasMatrixExt::matrix_prod
 * (mod.rs:1094, 1168, 1169, 1174), matrix_sum / row_vector_sum (mod.rs:1186-1189, 1203-1206,
 * 1214-1217), matrix_scale / row_vector_scale (mod.rs:1199-1202, 1359-1362).
 * C(m,n) = alpha * op(A) * op(B) + beta * C, all column-major; transX != 0 means transposed.
 * ------------------------------------------------------------------------------------------- */
/* Optional scratch (256-byte aligned): with it, GEMMs whose result has too few tiles to fill the
 * GPU split the contraction across blocks and reduce in a fixed order; without it (ws == NULL)
 * the same result is computed unsplit. */
size_t rh_sgemm_workspace_bytes(int32_t m, int32_t n, int32_t k);
/* Largest need when one extent varies from 1 up to the value given (which: 0 = m, 1 = n, 2 = k): the affine
 * operators call with the batch as n (forward, data gradient) or k (weight gradient) and any batch <= batch_cap. */
size_t rh_sgemm_workspace_bytes_upto(int32_t m, int32_t n, int32_t k, int which);
int rh_sgemm(int transA, int transB, int32_t m, int32_t n, int32_t k, float alpha, const float* A,
             int32_t lda, const float* B, int32_t ldb, float beta, float* C, int32_t ldc, void* ws,
             size_t ws_bytes, int flags, rh_stream_t stream);
/* rh_sgemm followed, in the same pass over C, by what AffineOperator::forward does next (mod.rs:1168-1176: matrix_prod,
 * then the bias row added to every column of the (out, batch) result, then the activation): with RH_FUSE_BIAS in `flags`,
 * bias[i], i < m, is added to C(i, j) after the alpha/beta blend; with RH_FUSE_RELU the result is then clamped at 0.
 * Each element goes through the same roundings as in the three separate calls. */
int rh_sgemm_bias_act(int transA, int transB, int32_t m, int32_t n, int32_t k, float alpha, const float* A,
                      int32_t lda, const float* B, int32_t ldb, float beta, float* C, int32_t ldc, const float* bias,
                      void* ws, size_t ws_bytes, int flags, rh_stream_t stream);
int rh_saxpy(int64_t n, float alpha, const float* x, float* y, rh_stream_t stream);
int rh_sscal(int64_t n, float alpha, float* x, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Pooling.  Replaces CudnnPoolingOp::forward / ::backward (mod.rs:2103-2107, 2115-2121; modes
 * Max and AverageCountIncludingPadding, mod.rs:2061-2065; floor extent mod.rs:2022-2027) and the
 * gen-1 kernels rembrandt_kernel_image_{max,average}_pool{,_backward} with their ceil extent and
 * int32 arg-max mask (src/layer.rs:1741-1747, 1797-1813, 1824-1840).
 * opt_argmax (may be NULL): per output element the h*W+w index inside its input plane of the
 * selected tap (-1: window without in-range tap).  Backward overwrites dx; with opt_argmax
 * given it does not read x or y.
 * ------------------------------------------------------------------------------------------- */
enum { RH_POOL_MAX = 0, RH_POOL_AVG_INCL_PAD = 1 };
enum { RH_ROUND_FLOOR = 0, RH_ROUND_CEIL = 1 };
typedef struct {
  int32_t N, C, H, W;
  int32_t size, stride, pad;
  int32_t mode;  /* RH_POOL_* */
  int32_t round; /* RH_ROUND_* */
} rh_pool_geom;
int32_t rh_pool2d_out_dim(int32_t in, int32_t size, int32_t stride, int32_t pad, int32_t round);
int rh_pool2d_fwd(const rh_pool_geom* g, const float* x, float* y, int32_t* opt_argmax,
                  rh_stream_t stream);
int rh_pool2d_bwd(const rh_pool_geom* g, const float* x, const float* y, const float* dy, float* dx,
                  const int32_t* opt_argmax, rh_stream_t stream);
/* Max-pool backward with the backward mask of the ReLU that produced x folded in (the pair K9' + K4 of
 * Pool2dOperator::backward followed by the producer's rect_backprop, src/operator/mod.rs:2113-2121, 1731-1738):
 * dx = [x > 0] * pool_bwd(dy).  x is not read: an arg-max element carries x = y, so windows with y <= 0 route
 * nothing.  Needs the arg-max mask of the forward pass; rh_pool2d_bwd_relu_supported says whether the geometry is
 * covered (else use rh_pool2d_bwd and the separate ReLU kernel). */
int rh_pool2d_bwd_relu_supported(const rh_pool_geom* g);
int rh_pool2d_bwd_relu(const rh_pool_geom* g, const float* y, const float* dy, float* dx, const int32_t* argmax,
                       rh_stream_t stream);
/* Average-pool backward with the same fold: dx = [x > 0] * pool_bwd(dy), x the pool's input (the ReLU's output);
 * bit-identical to rh_pool2d_bwd followed by rembrandt_kernel_batch_map_rect_backprop_inplace on dx.
 * RH_E_UNSUPPORTED for max pooling. */
int rh_pool2d_bwd_avg_relu(const rh_pool_geom* g, const float* x, const float* dy, float* dx, rh_stream_t stream);
/* The same pooling with a one-byte mask: slot[n,c,p,q] = r*size + s of the winning element inside its window (first
 * maximum, as above), 255 for a window without elements.  For an operator's private mask (a quarter of the int32
 * form's bytes on both passes; the gen-1 API's int32 plane index, src/layer.rs:1797-1813, stays rh_pool2d_fwd's).
 * rh_pool2d_slot_supported: nonzero for the geometries that have this form (max pooling, size <= 15, planes that fit the
 * LDS kernels).  rh_pool2d_bwd_slot: dx from dy and the slots; with relu_y (the pooled outputs) it also applies the
 * backward mask of the ReLU that produced x, as rh_pool2d_bwd_relu does. */
int rh_pool2d_slot_supported(const rh_pool_geom* g);
int rh_pool2d_fwd_slot(const rh_pool_geom* g, const float* x, float* y, uint8_t* slot, rh_stream_t stream);
int rh_pool2d_bwd_slot(const rh_pool_geom* g, const float* relu_y, const float* dy, float* dx, const uint8_t* slot,
                       rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Softmax / KL loss / reductions.  rh_softmax_fwd replaces CudnnSoftmaxOp::forward
 * (src/operator/loss.rs:121-126); the rembrandt_kernel_* symbols keep the rembrandt_kernels::ffi
 * names and argument lists seen at loss.rs:132-140, 191-200, 203-210, 229-239.  The reference
 * asserts len <= 1024 for the block reductions; these kernels have no such limit.
 * ------------------------------------------------------------------------------------------- */
int rh_softmax_fwd(const float* x, float* p, int32_t C, int32_t N, rh_stream_t stream);
void rembrandt_kernel_batch_map_softmax_kl_backward(const float* p, int32_t C, int32_t N,
                                                    const int32_t* labels, const float* weights,
                                                    float* dx, rh_stream_t stream);
void rembrandt_kernel_batch_map_softmax_kl_loss1(const float* p, int32_t C, int32_t N,
                                                 const int32_t* labels, const float* weights,
                                                 float beta, float* loss1, rh_stream_t stream);
void rembrandt_kernel_batch_blockreduce_sum(const float* src, int32_t len, int32_t batch,
                                            float* dst, float beta, rh_stream_t stream);
void rembrandt_kernel_batch_blockreduce_argmax(const float* src, int32_t len, int32_t batch,
                                               float* max_out, int32_t* idx_out,
                                               rh_stream_t stream);
/* The five calls above as one launch, for a train step (SgdOpt::train, src/opt/sgd/new.rs:383-420: forward,
 * store_output_categories, store_loss, then backward starts with the loss operator): p = softmax(x) (N rows of C),
 * max_out / idx_out = row maximum and lowest arg-max of p, loss1[n] = -weights[n] log p[n, labels[n]],
 * loss_sum[0] = sum_n loss1[n], dx[n, c] = weights[n] (p[n, c] - [c == labels[n]]).  Bit-identical to the separate
 * calls.  `counter` is one device word that is zero before the first call; every call leaves it zero. */
int rh_softmax_kl_step(const float* x, int32_t C, int32_t N, const int32_t* labels, const float* weights, float* p,
                       float* max_out, int32_t* idx_out, float* loss1, float* loss_sum, float* dx, uint32_t* counter,
                       rh_stream_t stream);

/* The classifier tail of a train step in two launches: AffineOperator::forward of two layers (mod.rs:1168-1176; the
 * first with ReLU or identity, the second with identity), the loss operator's step above (loss.rs:118-240), and the
 * backward passes of the two layers (mod.rs:1186-1217).  Weights are the reference's column-major (in, out) = [out][in],
 * activations [sample][channel].
 *   rh_affine2_softmax_kl_step   h = act(W1 x + b1) (B x H), logits = W2 h + b2 (B x C), then p, max_out, idx_out, loss1,
 *                                loss_sum, dlogits exactly as rh_softmax_kl_step's p .. dx, and the data gradients
 *                                dh = [h > 0] * W2^T dlogits (the first layer's delta after its activation's backward)
 *                                and, where dx is not NULL, dx = W1^T dh.  One block per sample.  `counter` as above.
 *   rh_affine2_bwd_params        dW1 = dh^T x, db1 = sum_n dh, dW2 = dlogits^T h, db2 = sum_n dlogits, each
 *                                out = sum + beta * out (beta 0: out is not read).
 *   rh_affine2_softmax_kl_step_supported   1 where the sizes have this form (a sample's chain in one block's LDS:
 *                                I <= 4096, H <= 2048, C <= 64, I * H <= 2^17, B * I * H <= 2^26: every block reads the
 *                                first layer's weights), else both return
 *                                RH_E_UNSUPPORTED.
 * With I = 0 and x = NULL both start from an h that is already there (a first layer too large for this form, whose
 * products stay with rh_sgemm): rh_affine2_softmax_kl_step then reads h, writes logits .. dh and leaves dx alone (w1, b1
 * unused); rh_affine2_bwd_params forms dW2 and db2 (dw1 unused) and, where db1 is not NULL, db1 = sum_n dh + beta1 * db1.
 * Sums are taken in a fixed order that differs from the tiled products': results agree with the separate calls to
 * rounding, not bit for bit. */
int rh_affine2_softmax_kl_step_supported(int32_t B, int32_t I, int32_t H, int32_t C);
int rh_affine2_softmax_kl_step(int32_t B, int32_t I, int32_t H, int32_t C, int32_t relu1, const float* x, const float* w1,
                               const float* b1, const float* w2, const float* b2, const int32_t* labels,
                               const float* weights, float* h, float* logits, float* p, float* max_out, int32_t* idx_out,
                               float* loss1, float* loss_sum, float* dlogits, float* dh, float* dx, uint32_t* counter,
                               rh_stream_t stream);
int rh_affine2_bwd_params(int32_t B, int32_t I, int32_t H, int32_t C, const float* x, const float* h, const float* dh,
                          const float* dlogits, float beta1, float* dw1, float* db1, float beta2, float* dw2, float* db2,
                          rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * SGD.  rh_sgd_momentum_step is the fused form of the BLAS-1 sequence regularize ->
 * accumulate_grads -> update_params -> reset (mod.rs:1178-1218, 1355-1363; driven by
 * src/opt/sgd/new.rs:345-495):  g += l2*W (if l2 > 0); v = mu*v; v += scale*g; W += apply*v;
 * g = 0 (if zero_grad).  rh_descend is the gen-1/gen-2 update g += l2*W; W -= s*g
 * (src/layer_new.rs:596-617, src/layer.rs:1710-1715).
 * ------------------------------------------------------------------------------------------- */
int rh_sgd_momentum_step(int64_t n, float* W, float* g, float* v, float l2, float scale, float mu,
                         float apply, int zero_grad, rh_stream_t stream);
/* rh_sgd_momentum_step over several tensors in one launch (`tensors` is a host array; each entry carries its own l2,
 * as the batch-normalised operators decay their filters only, src/operator/conv.rs:647): what one `update` fan-out
 * over a chain of operators (src/operator/worker.rs:420-445) issues, without a launch per parameter block.  Same
 * arithmetic per element as rh_sgd_momentum_step. */
typedef struct rh_sgd_tensor {
  float* W;
  float* g;
  float* v;
  int64_t n;
  float l2;
  int32_t keep_grad;   /* nonzero: leave g as it is even with zero_grad (the caller overwrites it, beta = 0, next time) */
} rh_sgd_tensor;
int rh_sgd_momentum_step_multi(int32_t count, const rh_sgd_tensor* tensors, float scale, float mu, float apply,
                               int zero_grad, rh_stream_t stream);
int rh_descend(int64_t n, float* W, float* g, float s, float l2, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Input preprocessing of Data3dOperator::forward (src/operator/mod.rs:640-790) and dropout
 * (src/operator/mod.rs:2211-2248).  The three `rembrandt_kernel_*` symbols keep the names and argument
 * lists of the reference's call sites; their bodies live in a crate outside its tree, so what they compute
 * is this build's reading of those call sites:
 *   rh_crop_nchw                 replaces CudnnTransformOp::transform on a strided 4-d view (mod.rs:666-691):
 *                                dst[p][h][w] = src[p][off_h + h][off_w + w], p < planes = batch * channels.
 *   ..._blockmap256_flip         dst[r][w] = src[r][width-1-w], r < rows (mod.rs:767-773); no width <= 256 limit.
 *   ..._preproc_pca3_noise       dst[n][c][i] = src[n][c][i] + sum_j svecs[3j + c] * alphas[3n + j] * svals[j]
 *                                (3 channels; mod.rs:716-725).
 *   rembrandt_kernel_map_dropout mask[i] = rnd[i] > drop_ratio; out[i] = mask ? scale * in[i] : 0 (mod.rs:2221-2229).
 *   ..._map_dropout_backprop     in_delta[i] = mask[i] ? scale * out_delta[i] : 0 (mod.rs:2239-2246).
 * ------------------------------------------------------------------------------------------- */
int rh_crop_nchw(const float* src, float* dst, int64_t planes, int32_t in_w, int32_t in_h, int32_t crop_w,
                 int32_t crop_h, int32_t off_w, int32_t off_h, rh_stream_t stream);
void rembrandt_kernel_batch_blockmap256_flip(const float* src, int32_t width, int32_t rows, float* dst,
                                             rh_stream_t stream);
void rembrandt_kernel_batch_map_preproc_pca3_noise(const float* src, int32_t spatial, int32_t batch,
                                                   const float* alphas, const float* svals, const float* svecs,
                                                   float* dst, rh_stream_t stream);
void rembrandt_kernel_map_dropout(const float* in, int32_t n, float drop_ratio, float scale, const float* rnd,
                                  float* out, int32_t* mask, rh_stream_t stream);
void rembrandt_kernel_map_dropout_backprop(const float* out_delta, int32_t n, float drop_ratio, float scale,
                                           const int32_t* mask, float* in_delta, rh_stream_t stream);

/* Cross-channel local response normalisation (the `local_res_norm` layer type of the reference's `.model`
 * grammar, examples/imagenet_alexnet.model:31-37; the reference's own layer is an empty stub,
 * src/layer.rs:1846-1899, so the arithmetic is the published one those parameters name):
 *   d[n,c,h,w] = min_div + scale * sum_{c' = c - size/2 .. c + (size-1)/2, clipped} x[n,c',h,w]^2
 *   y = x * d^-power.   `denom` (same shape as x) receives d and is an input of the backward pass. */
typedef struct rh_lrn_geom {
  int32_t N, C, H, W;
  int32_t size;
  float scale, power, min_div;
} rh_lrn_geom;
int rh_lrn_fwd(const rh_lrn_geom* g, const float* x, float* y, float* denom, rh_stream_t stream);
int rh_lrn_bwd(const rh_lrn_geom* g, const float* x, const float* y, const float* denom, const float* dy, float* dx,
               rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Spatial batch normalisation, NCHW fp32, `plane` = H*W.  Replaces CudnnBatchNormOp in
 * cudnnBatchNormMode_t::Spatial (constructed at src/operator/conv.rs:225-232; forward_inference :493-506,
 * forward_training :520-535, backward :594-607).  With m = N*plane values per channel:
 *   mean_c = sum(x)/m,  ivar_c = 1/sqrt(sum((x-mean_c)^2)/m + epsilon)
 *   forward_training:  y = alpha*(scale_c*(x-mean_c)*ivar_c + bias_c) + beta*y
 *                      cached_mean = mean, cached_ivar = ivar,
 *                      running_mean = (1-ema_factor)*running_mean + ema_factor*mean
 *                      running_ivar = (1-ema_factor)*running_ivar + ema_factor*ivar
 *   forward_inference: the same map with (running_mean, running_ivar) in place of the batch statistics
 *   backward:          dscale_c = beta_param*dscale_c + alpha_param*sum(dy*xhat),  xhat = (x-cached_mean)*cached_ivar
 *                      dbias_c  = beta_param*dbias_c  + alpha_param*sum(dy)
 *                      dx = alpha_data*scale_c*cached_ivar*(dy - sum(dy)/m - xhat*sum(dy*xhat)/m) + beta_data*dx
 * The moving "ivar" is an average of inverse standard deviations, as the reference's buffer names
 * (bn_running_ivar, initialised to 1) say; what cuDNN v4 kept in that buffer cannot be checked here.
 * RH_FUSE_RELU (forward only) clamps the blended result at 0: the in-place ReLU that follows the call in the
 * reference (src/operator/conv.rs:538-551).  `ws` needs rh_bnorm_workspace_bytes(N, C, plane) bytes. */
size_t rh_bnorm_workspace_bytes(int N, int C, int plane);
size_t rh_bnorm_workspace_bytes_upto(int N, int C, int plane); /* largest need of N' = 1..N */
int rh_bnorm_fwd_train(int N, int C, int plane, float alpha, const float* x, float beta, float* y, double ema_factor,
                       double epsilon, const float* scale, const float* bias, float* running_mean, float* running_ivar,
                       float* cached_mean, float* cached_ivar, void* ws, size_t ws_bytes, int flags, rh_stream_t stream);
int rh_bnorm_fwd_infer(int N, int C, int plane, float alpha, const float* x, float beta, float* y, double epsilon,
                       const float* scale, const float* bias, const float* running_mean, const float* running_ivar,
                       void* ws, size_t ws_bytes, int flags, rh_stream_t stream);
int rh_bnorm_bwd(int N, int C, int plane, float alpha_data, float beta_data, const float* x, const float* dy, float* dx,
                 float alpha_param, float beta_param, double epsilon, const float* scale, float* dscale, float* dbias,
                 const float* cached_mean, const float* cached_ivar, void* ws, size_t ws_bytes, rh_stream_t stream);
/* rh_bnorm_bwd preceded by the backward of the ReLU that rh_bnorm_fwd_train fused (flags RH_FUSE_RELU, alpha 1, beta 0):
 * dy counts only where the forward output was positive.  Replaces the pair the reference issues, its in-place ReLU
 * backward kernel on the delta followed by the batch-norm backward (src/operator/conv.rs:577-607), without the pass
 * over the delta: the sign of the forward output is recomputed from x, the cached statistics, `scale` and `bias`
 * by the forward pass's own expression, so `scale` and `bias` must still hold the forward pass's values. */
int rh_bnorm_bwd_relu(int N, int C, int plane, float alpha_data, float beta_data, const float* x, const float* dy, float* dx,
                      float alpha_param, float beta_param, double epsilon, const float* scale, const float* bias,
                      float* dscale, float* dbias, const float* cached_mean, const float* cached_ivar, void* ws,
                      size_t ws_bytes, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Host-side seeded generator for synthetic inputs and parameter initialisation (stands in for
 * the rng crate's Xorshiftplus128Rng + rand 0.3 distributions of src/operator/mod.rs:964-1006,
 * 1554-1592, whose bit streams cannot be reproduced).  Element i of stream (seed, stream_id) is
 * a pure function of (seed, stream_id, i).  Host pointers.
 * ------------------------------------------------------------------------------------------- */
int rh_rng_fill_uniform(uint64_t seed, uint64_t stream_id, float* host, size_t n, float lo, float hi);
int rh_rng_fill_normal(uint64_t seed, uint64_t stream_id, float* host, size_t n, float mean, float std);
int rh_rng_fill_int(uint64_t seed, uint64_t stream_id, int32_t* host, size_t n, int32_t modulus);
/* Device form: dst[i] (device pointer) = element (first + i) of rh_rng_fill_uniform(seed, stream_id, ., ., 0, 1),
 * bit for bit.  Stands in for DeviceBuffer::sample(&UniformDist) (mod.rs:2220). */
int rh_rng_fill_uniform01_device(uint64_t seed, uint64_t stream_id, uint64_t first, float* dst, size_t n,
                                 rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Packed bf16 activations for forward-only chains (RH_MATH_BF16_MFMA_FP32ACC without its per-call conversions; no
 * counterpart in the reference, whose inference pass, OpPhase::Inference in src/operator/mod.rs:1663-1718, is the fp32
 * forward).  A packed activation tensor holds bf16 values as [n][H + 2*halo][C/8][W + 2*halo][8] (C a multiple of 8;
 * rh_bf16_act_bytes), with a zero border of `halo` elements that the producer never writes: zero the buffer once.  It is
 * what the bf16 convolution's loaders read when halo equals that convolution's padding, so a producer that writes it
 * (the convolution below, or a max-pool between them) removes the consumer's fp32 -> bf16 pass and halves the
 * producer's store.  Values are the fp32 results rounded to nearest even, i.e. exactly what the consumer of an fp32
 * activation would have rounded them to (ReLU and max commute with the rounding), so a chain run this way is
 * bit-identical to the same chain through rh_conv2d_fwd(..., RH_MATH_BF16_MFMA_FP32ACC) on fp32 activations.
 *   rh_bf16_pack_nchw / rh_bf16_unpack_nchw   fp32 NCHW <-> packed (unpack gives the bf16 values as fp32).
 *   rh_conv2d_fwd_bf16_filter_bytes           size of a convolution's converted filter (0: the geometry has no packed
 *                                             form); rh_conv2d_fwd_bf16_prep_filter fills it (256-byte aligned).  It
 *                                             stays valid until the weights change.
 *   rh_conv2d_fwd_bf16_takes_packed           nonzero if the geometry reads a packed input (input channels a multiple
 *                                             of 8); otherwise pass the fp32 image `x`.
 *   rh_conv2d_fwd_bf16_packed                 y = conv(x, w) (+ bias) (ReLU) from exactly one of `xp` (packed, halo =
 *                                             g->pad) and `x` (fp32 NCHW, converted into `ws` of
 *                                             rh_conv2d_fwd_bf16_workspace_bytes), to exactly one of `y` (fp32 NCHW) and
 *                                             `yp` (packed with halo yp_halo; K a multiple of 8).  flags: RH_FUSE_*;
 *                                             RH_ALGO_SCALAR_OFFSET takes the streaming 1x1 kernel wherever it can run
 *                                             (tests: the same bits as the kernel chosen by default).
 *   rh_pool2d_fwd_bf16_packed                 max pooling from a packed input (halo 0) to a packed output.
 * ------------------------------------------------------------------------------------------- */
size_t rh_bf16_act_bytes(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo);
int rh_bf16_pack_nchw(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo, const float* x, void* xp,
                      rh_stream_t stream);
int rh_bf16_unpack_nchw(int32_t N, int32_t C, int32_t H, int32_t W, int32_t halo, const void* xp, float* x,
                        rh_stream_t stream);
size_t rh_conv2d_fwd_bf16_filter_bytes(const rh_conv_geom* g);
int rh_conv2d_fwd_bf16_takes_packed(const rh_conv_geom* g);
size_t rh_conv2d_fwd_bf16_workspace_bytes(const rh_conv_geom* g);
int rh_conv2d_fwd_bf16_prep_filter(const rh_conv_geom* g, const float* w, void* wprep, size_t wprep_bytes,
                                   rh_stream_t stream);
int rh_conv2d_fwd_bf16_packed(const rh_conv_geom* g, const void* xp, const float* x, const void* wprep,
                              const float* bias, float* y, void* yp, int32_t yp_halo, void* ws, size_t ws_bytes,
                              int flags, rh_stream_t stream);
int rh_pool2d_fwd_bf16_packed(const rh_pool_geom* g, const void* xp, void* yp, int32_t yp_halo, rh_stream_t stream);

/* ---------------------------------------------------------------------------------------------
 * Per-launch timing (no counterpart in the reference, which only takes wall-clock laps around
 * minibatches, src/opt/sgd/new.rs:273-274).  While enabled, every kernel launch of this library is
 * bracketed by HIP events on its stream.  Record i = {kernel tag, algorithmic work (FLOPs for the
 * MFMA contractions, bytes for the bandwidth-bound kernels), elapsed milliseconds}.
 * ------------------------------------------------------------------------------------------- */
int rh_profile_enable(int on);
int rh_profile_enabled(void);
/* Record only launches whose tag starts with `prefix` (NULL or "" = all).  Set it while disabled. */
int rh_profile_filter(const char* prefix);
int rh_profile_count(void);
int rh_profile_get(int i, const char** tag, double* work, float* ms);
int rh_profile_reset(void);

/* Calibration launches for the roofline report (no counterpart in the reference): a register-only
 * fp32 MFMA loop (blocks x 4 waves, each issuing iters * nacc MFMAs, nacc in {4, 8}; FLOPs =
 * blocks * 4 * iters * nacc * 4096) and a float4 copy of n floats (bytes = 8 * n). */
int rh_probe_mfma_loop(int blocks, int nacc, int iters, float* sink, rh_stream_t stream);
/* The same loop on operands that differ per lane and per instruction (realistic data toggling and power draw). */
int rh_probe_mfma_loop_varied(int blocks, int iters, float* sink, rh_stream_t stream);
int rh_probe_copy(const float* src, float* dst, size_t n, rh_stream_t stream);
#ifdef __cplusplus
}
#endif
#endif /* REMBRANDT_HIP_H */
