// Host-side operator layer (see operator.hpp).  Uses only the C ABI of rembrandt_hip.h.
#include "operator.hpp"

#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>

namespace rembrandt {

void panic(const std::string& msg) { throw std::runtime_error(msg); }

void unwrap(int code, const char* what) {
  if (code != 0) panic(std::string(what) + " failed: " + std::to_string(code) + " (" + rh_error_string(code) + ")");
}

static void unwrap_last(const char* what) { unwrap(rh_last_error(), what); }

#define RB_ASSERT(cond) \
  do { if (!(cond)) ::rembrandt::panic(std::string("assertion failed: ") + #cond); } while (0)

DeviceContext::DeviceContext(int device_idx) : ctx_(nullptr) { unwrap(rh_ctx_create(device_idx, &ctx_), "rh_ctx_create"); }
DeviceContext::~DeviceContext() { rh_ctx_destroy(ctx_); }
void DeviceContext::sync() const { unwrap(rh_ctx_sync(ctx_), "rh_ctx_sync"); }
PinnedBytes::PinnedBytes(size_t len, std::shared_ptr<DeviceContext> ctx) : len_(len), ctx_(std::move(ctx)) {
  void* p = nullptr;
  unwrap(rh_host_malloc(ctx_->raw(), len, &p), "rh_host_malloc");
  ptr_ = static_cast<uint8_t*>(p);
}
PinnedBytes::~PinnedBytes() { rh_host_free(ctx_->raw(), ptr_); }

rh_stream_t DeviceContext::aux_stream() const {
  rh_stream_t s = rh_ctx_aux_stream(ctx_);
  if (!s) panic("rh_ctx_aux_stream failed");
  return s;
}
void DeviceContext::fork() const { unwrap(rh_ctx_fork(ctx_), "rh_ctx_fork"); }
void DeviceContext::join() const { unwrap(rh_ctx_join(ctx_), "rh_ctx_join"); }
void DeviceContext::begin_capture() const { unwrap(rh_ctx_begin_capture(ctx_), "rh_ctx_begin_capture"); }
rh_graph* DeviceContext::end_capture() const {
  rh_graph* g = nullptr;
  unwrap(rh_ctx_end_capture(ctx_, &g), "rh_ctx_end_capture");
  return g;
}
void DeviceContext::abort_capture() const { (void)rh_ctx_end_capture(ctx_, nullptr); }
void DeviceContext::launch(rh_graph* g) const { unwrap(rh_graph_launch(g, ctx_), "rh_graph_launch"); }

// ---- configs ----------------------------------------------------------------------------------------
static size_t out_dim_floor(size_t in, size_t size, size_t stride, size_t pad) {
  // max(0, in + 2*pad - size + stride) / stride   (src/operator/mod.rs:1393-1398, 2022-2027)
  const long long t = (long long)in + 2 * (long long)pad - (long long)size + (long long)stride;
  return (size_t)(std::max<long long>(0, t) / (long long)stride);
}

Dims3 Conv2dOperatorConfig::get_out_dims() const {
  return {out_dim_floor(in_dims.w, conv_size, conv_stride, conv_pad),
          out_dim_floor(in_dims.h, conv_size, conv_stride, conv_pad), out_channels};
}

Dims3 BNormConv2dOperatorConfig::get_out_dims() const {
  return {out_dim_floor(in_dims.w, conv_size, conv_stride, conv_pad),
          out_dim_floor(in_dims.h, conv_size, conv_stride, conv_pad), out_channels};
}

Dims3 Pool2dOperatorConfig::get_out_dims() const {
  const int r = ceil_mode ? RH_ROUND_CEIL : RH_ROUND_FLOOR;
  return {(size_t)rh_pool2d_out_dim((int)in_dims.w, (int)pool_size, (int)pool_stride, (int)pool_pad, r),
          (size_t)rh_pool2d_out_dim((int)in_dims.h, (int)pool_size, (int)pool_stride, (int)pool_pad, r), in_dims.c};
}

Dims3 Data3dOperatorConfig::get_out_dims() const {
  Dims3 out = in_dims;
  for (const auto& p : preprocs) {
    if (p.kind == Data3dPreproc::Crop) {
      if (p.crop_width > out.w || p.crop_height > out.h) panic("assertion failed: crop fits the frame");
      out = {p.crop_width, p.crop_height, out.c};
    }
  }
  return out;
}

// ---- NdArray blobs ----------------------------------------------------------------------------------
void ndarray_serialize(std::vector<uint8_t>& out, const float* data, const size_t* dims, size_t ndim) {
  const uint8_t magic[4] = {'N', 'D', 0, 1};
  out.insert(out.end(), magic, magic + 4);
  const uint32_t nd = (uint32_t)ndim;
  for (int b = 0; b < 4; ++b) out.push_back((uint8_t)(nd >> (8 * b)));
  size_t count = 1;
  for (size_t i = 0; i < ndim; ++i) {
    const uint64_t d = dims[i];
    for (int b = 0; b < 8; ++b) out.push_back((uint8_t)(d >> (8 * b)));
    count *= dims[i];
  }
  const uint8_t* bytes = reinterpret_cast<const uint8_t*>(data);  // little-endian host
  out.insert(out.end(), bytes, bytes + count * sizeof(float));
}

size_t ndarray_deserialize(const uint8_t* blob, size_t len, std::vector<size_t>* dims, std::vector<float>* data) {
  if (len < 8 || blob[0] != 'N' || blob[1] != 'D' || blob[2] != 0 || blob[3] != 1) panic("NdArray: bad magic");
  uint32_t nd = 0;
  for (int b = 0; b < 4; ++b) nd |= (uint32_t)blob[4 + b] << (8 * b);
  if (nd == 0 || nd > 8 || len < 8 + 8 * (size_t)nd) panic("NdArray: bad rank or truncated header");
  dims->clear();
  size_t count = 1, off = 8;
  for (uint32_t i = 0; i < nd; ++i, off += 8) {
    uint64_t d = 0;
    for (int b = 0; b < 8; ++b) d |= (uint64_t)blob[off + b] << (8 * b);
    if (d != 0 && count > (size_t)1 << 40) panic("NdArray: dimensions overflow");
    dims->push_back((size_t)d);
    count *= (size_t)d;
  }
  if (len - off < count * sizeof(float)) panic("NdArray: truncated data");
  data->resize(count);
  if (count) std::memcpy(data->data(), blob + off, count * sizeof(float));
  return off + count * sizeof(float);
}

size_t OperatorConfig::params_len() const {
  switch (kind) {
    case Affine: return affine.params_len();
    case Conv2d: return conv2d.params_len();
    case BNormConv2d: return bnorm_conv2d.params_len();
    case StackResConv2d: return stack_res_conv2d.params_len();
    case ProjStackResConv2d: return proj_stack_res_conv2d.params_len();
    default: return 0;
  }
}

size_t SequentialOperatorConfig::params_len() const {
  size_t n = 0;
  for (const auto& op : hidden_ops) n += op.params_len();
  return n;
}
SequentialOperatorConfig& SequentialOperatorConfig::data3d(const Data3dOperatorConfig& cfg) {
  input_op = OperatorConfig();
  input_op.kind = OperatorConfig::Data3d;
  input_op.data3d = cfg;
  has_input = true;
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::affine(const AffineOperatorConfig& cfg) {
  OperatorConfig c = OperatorConfig();
  c.kind = OperatorConfig::Affine;
  c.affine = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::conv2d(const Conv2dOperatorConfig& cfg) {
  OperatorConfig c = OperatorConfig();
  c.kind = OperatorConfig::Conv2d;
  c.conv2d = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::pool2d(const Pool2dOperatorConfig& cfg) {
  OperatorConfig c = OperatorConfig();
  c.kind = OperatorConfig::Pool2d;
  c.pool2d = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::dropout(const DropoutOperatorConfig& cfg) {
  OperatorConfig c = OperatorConfig();
  c.kind = OperatorConfig::Dropout;
  c.dropout = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::local_res_norm(const LocalResNormOperatorConfig& cfg) {
  OperatorConfig c = OperatorConfig();
  c.kind = OperatorConfig::LocalResNorm;
  c.lrn = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::bnorm_conv2d(const BNormConv2dOperatorConfig& cfg) {
  OperatorConfig c{};
  c.kind = OperatorConfig::BNormConv2d;
  c.bnorm_conv2d = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::stack_res_conv2d(const StackResConv2dOperatorConfig& cfg) {
  OperatorConfig c{};
  c.kind = OperatorConfig::StackResConv2d;
  c.stack_res_conv2d = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::proj_stack_res_conv2d(const ProjStackResConv2dOperatorConfig& cfg) {
  OperatorConfig c{};
  c.kind = OperatorConfig::ProjStackResConv2d;
  c.proj_stack_res_conv2d = cfg;
  hidden_ops.push_back(c);
  return *this;
}
SequentialOperatorConfig& SequentialOperatorConfig::softmax_kl_loss(const CategoricalLossConfig& cfg) {
  loss_op = OperatorConfig();
  loss_op.kind = OperatorConfig::SoftmaxKLLoss;
  loss_op.loss = cfg;
  has_loss = true;
  return *this;
}

// ---- parameter block shared by Affine and Conv2d -----------------------------------------------------
namespace {

typedef std::shared_ptr<DeviceContext> Ctx;

// Scratch is allocated once for batch_cap, but a pass may be called with any batch <= batch_cap and the library's
// plans are not monotone in the batch (fewer result tiles make it cut the contraction into more slices, whose partial
// sums can need more room than the full batch does): every scratch buffer is sized with the *_upto functions.
size_t conv_ws_upto(const rh_conv_geom& g, int pass) { return rh_conv2d_workspace_bytes_upto(&g, pass); }
size_t bias_ws_upto(int batch, int K, int plane) { return rh_conv2d_bwd_bias_workspace_bytes_upto(batch, K, plane); }
size_t bnorm_ws_upto(int batch, int C, int plane) { return rh_bnorm_workspace_bytes_upto(batch, C, plane); }
// The affine GEMMs of a layer (out, B, in), (in, out, B), (in, B, out): B is the batch.
size_t sgemm_ws_upto(int m, int n, int k, int batch_dim /* 1 = n is the batch, 2 = k is */, int /*batch*/) {
  return rh_sgemm_workspace_bytes_upto(m, n, k, batch_dim);
}

struct ParamTensors {
  std::unique_ptr<DeviceBuffer<float>> weights, bias;
  // backward-capable operators only
  std::unique_ptr<DeviceBuffer<float>> grad_weights, grad_bias, acc_grad_weights, acc_grad_bias, save_weights, save_bias;
  size_t wlen = 0, blen = 0;
  size_t wrows = 0, wcols = 0;  // bound of the weights as the reference's Array2d: (in or R*S*C, out), first index fastest
  Ctx ctx;
  // The fused SGD step would write 4 bytes of zero per parameter into the gradient, and the next backward pass would
  // read them back to add to (beta = 1).  Instead the step leaves the gradient buffers as they are and marks them
  // stale: they stand for zeros.  The next backward pass then overwrites (beta = 0); anything else that looks at the
  // gradients first makes the zeros real (touch_grads).
  bool grads_stale = false;
  void touch_grads() {
    if (!grads_stale) return;
    grads_stale = false;
    unwrap(rh_memset_f32(grad_weights->as_mut_ptr(), 0.0f, wlen, s()), "set_constant");
    unwrap(rh_memset_f32(grad_bias->as_mut_ptr(), 0.0f, blen, s()), "set_constant");
  }
  // beta of the gradient accumulation of one backward pass (weights and bias alike); the buffers are real afterwards
  float take_backward_beta() {
    const float b = grads_stale ? 0.0f : 1.0f;
    grads_stale = false;
    return b;
  }

  void alloc(size_t wl, size_t bl, bool backward, Ctx c) {
    wlen = wl; blen = bl; ctx = c;
    wcols = bl; wrows = bl ? wl / bl : 0;
    weights.reset(new DeviceBuffer<float>(wl, c));
    bias.reset(new DeviceBuffer<float>(bl, c));
    if (backward) {
      grad_weights.reset(new DeviceBuffer<float>(wl, c));
      grad_bias.reset(new DeviceBuffer<float>(bl, c));
      acc_grad_weights.reset(new DeviceBuffer<float>(wl, c));
      acc_grad_bias.reset(new DeviceBuffer<float>(bl, c));
      save_weights.reset(new DeviceBuffer<float>(wl, c));
      save_bias.reset(new DeviceBuffer<float>(bl, c));
    }
  }
  bool has_backward() const { return (bool)grad_weights; }
  rh_stream_t s() const { return ctx->stream(); }

  // g += l2*W for weights *and bias* (src/operator/mod.rs:1178-1193, 1797-1812)
  void regularize(Regularization reg) {
    RB_ASSERT(has_backward());
    RB_ASSERT(reg.l2_reg_coef >= 0.0f);
    touch_grads();
    if (reg.l2_reg_coef > 0.0f) {
      unwrap(rh_saxpy((int64_t)wlen, reg.l2_reg_coef, weights->as_ptr(), grad_weights->as_mut_ptr(), s()), "matrix_sum");
      unwrap(rh_saxpy((int64_t)blen, reg.l2_reg_coef, bias->as_ptr(), grad_bias->as_mut_ptr(), s()), "row_vector_sum");
    }
  }
  // v = momentum*v; v += scale*g (src/operator/mod.rs:1195-1207)
  void accumulate_grads(float scale, float momentum) {
    RB_ASSERT(has_backward());
    touch_grads();
    unwrap(rh_sscal((int64_t)wlen, momentum, acc_grad_weights->as_mut_ptr(), s()), "matrix_scale");
    unwrap(rh_sscal((int64_t)blen, momentum, acc_grad_bias->as_mut_ptr(), s()), "row_vector_scale");
    unwrap(rh_saxpy((int64_t)wlen, scale, grad_weights->as_ptr(), acc_grad_weights->as_mut_ptr(), s()), "matrix_sum");
    unwrap(rh_saxpy((int64_t)blen, scale, grad_bias->as_ptr(), acc_grad_bias->as_mut_ptr(), s()), "row_vector_sum");
  }
  // W += scale*v (src/operator/mod.rs:1210-1218)
  void update_params(float scale) {
    RB_ASSERT(has_backward());
    unwrap(rh_saxpy((int64_t)wlen, scale, acc_grad_weights->as_ptr(), weights->as_mut_ptr(), s()), "matrix_sum");
    unwrap(rh_saxpy((int64_t)blen, scale, acc_grad_bias->as_ptr(), bias->as_mut_ptr(), s()), "row_vector_sum");
  }
  // W += grad_scale*g + update_scale*v (src/operator/mod.rs:1220-1236)
  void update_params2(float grad_scale, float update_scale) {
    RB_ASSERT(has_backward());
    touch_grads();
    if (grad_scale != 0.0f) {
      unwrap(rh_saxpy((int64_t)wlen, grad_scale, grad_weights->as_ptr(), weights->as_mut_ptr(), s()), "matrix_sum");
      unwrap(rh_saxpy((int64_t)blen, grad_scale, grad_bias->as_ptr(), bias->as_mut_ptr(), s()), "row_vector_sum");
    }
    if (update_scale != 0.0f) {
      unwrap(rh_saxpy((int64_t)wlen, update_scale, acc_grad_weights->as_ptr(), weights->as_mut_ptr(), s()), "matrix_sum");
      unwrap(rh_saxpy((int64_t)blen, update_scale, acc_grad_bias->as_ptr(), bias->as_mut_ptr(), s()), "row_vector_sum");
    }
  }
  void save_params() {
    RB_ASSERT(has_backward());
    unwrap(rh_copy_d2d(save_weights->as_mut_ptr(), weights->as_ptr(), wlen * 4, s()), "send");
    unwrap(rh_copy_d2d(save_bias->as_mut_ptr(), bias->as_ptr(), blen * 4, s()), "send");
  }
  void restore_params() {
    RB_ASSERT(has_backward());
    unwrap(rh_copy_d2d(weights->as_mut_ptr(), save_weights->as_ptr(), wlen * 4, s()), "send");
    unwrap(rh_copy_d2d(bias->as_mut_ptr(), save_bias->as_ptr(), blen * 4, s()), "send");
  }
  // g *= 0 (src/operator/mod.rs:1355-1363)
  void reset() {
    if (!has_backward()) return;
    if (grads_stale) return;   // they already stand for zeros
    unwrap(rh_sscal((int64_t)wlen, 0.0f, grad_weights->as_mut_ptr(), s()), "matrix_scale");
    unwrap(rh_sscal((int64_t)blen, 0.0f, grad_bias->as_mut_ptr(), s()), "row_vector_scale");
  }
  // g += l2*W for weights and bias; W -= scale*g (src/layer_new.rs:596-617, 1133-1154)
  void descend(float scale, float l2, bool fused) {
    RB_ASSERT(has_backward());
    RB_ASSERT(l2 >= 0.0f);
    touch_grads();
    if (fused) {
      unwrap(rh_descend((int64_t)wlen, weights->as_mut_ptr(), grad_weights->as_mut_ptr(), scale, l2, s()), "rh_descend");
      unwrap(rh_descend((int64_t)blen, bias->as_mut_ptr(), grad_bias->as_mut_ptr(), scale, l2, s()), "rh_descend");
      return;
    }
    if (l2 > 0.0f) {
      unwrap(rh_saxpy((int64_t)wlen, l2, weights->as_ptr(), grad_weights->as_mut_ptr(), s()), "matrix_sum");
      unwrap(rh_saxpy((int64_t)blen, l2, bias->as_ptr(), grad_bias->as_mut_ptr(), s()), "row_vector_sum");
    }
    unwrap(rh_saxpy((int64_t)wlen, -scale, grad_weights->as_ptr(), weights->as_mut_ptr(), s()), "matrix_sum");
    unwrap(rh_saxpy((int64_t)blen, -scale, grad_bias->as_ptr(), bias->as_mut_ptr(), s()), "row_vector_sum");
  }
  // g *= scale (src/layer_new.rs:589-594, 1126-1131)
  void reset_gradients(float scale) {
    RB_ASSERT(has_backward());
    touch_grads();
    unwrap(rh_sscal((int64_t)wlen, scale, grad_weights->as_mut_ptr(), s()), "matrix_scale");
    unwrap(rh_sscal((int64_t)blen, scale, grad_bias->as_mut_ptr(), s()), "row_vector_scale");
  }
  void fused_sgd_step(float l2, float scale, float momentum, float apply, rh_stream_t st = nullptr) {
    RB_ASSERT(has_backward());
    if (!st) st = s();
    unwrap(rh_sgd_momentum_step((int64_t)wlen, weights->as_mut_ptr(), grad_weights->as_mut_ptr(),
                                acc_grad_weights->as_mut_ptr(), l2, scale, momentum, apply, 1, st), "rh_sgd_momentum_step");
    unwrap(rh_sgd_momentum_step((int64_t)blen, bias->as_mut_ptr(), grad_bias->as_mut_ptr(),
                                acc_grad_bias->as_mut_ptr(), l2, scale, momentum, apply, 1, st), "rh_sgd_momentum_step");
  }
  // Rows of one multi-tensor step: the gradients are read, not zeroed, and stand for zeros from then on.
  void sgd_tensors(float l2, std::vector<rh_sgd_tensor>& out) {
    RB_ASSERT(has_backward());
    touch_grads();   // (a step without a backward pass since the last one: the update must see zeros)
    out.push_back({weights->as_mut_ptr(), grad_weights->as_mut_ptr(), acc_grad_weights->as_mut_ptr(), (int64_t)wlen, l2, 1});
    out.push_back({bias->as_mut_ptr(), grad_bias->as_mut_ptr(), acc_grad_bias->as_mut_ptr(), (int64_t)blen, l2, 1});
    grads_stale = true;
  }
  // Host-side sampling in memory order, then a blocking H2D copy (src/operator/mod.rs:964-1006, 1554-1592).
  void init(const ParamsInit& init, const uint64_t seed[2], size_t fan_in, size_t fan_out, bool xavier_ok, const char* who) {
    std::vector<float> w(wlen);
    switch (init.kind) {
      case ParamsInit::Disabled: panic(std::string(who) + ": params init explicitly disabled");
      case ParamsInit::Uniform:
        unwrap(rh_rng_fill_uniform(seed[0], seed[1], w.data(), wlen, -init.value, init.value), "rh_rng_fill_uniform");
        break;
      case ParamsInit::Normal:
        unwrap(rh_rng_fill_normal(seed[0], seed[1], w.data(), wlen, 0.0f, init.value), "rh_rng_fill_normal");
        break;
      case ParamsInit::Xavier: {
        if (!xavier_ok) panic(std::string(who) + ": Xavier init is unimplemented for this operator");
        const float h = (float)std::sqrt(6.0 / (double)(fan_in + fan_out));
        unwrap(rh_rng_fill_uniform(seed[0], seed[1], w.data(), wlen, -h, h), "rh_rng_fill_uniform");
        break;
      }
      case ParamsInit::KaimingFwd: {
        const float sd = (float)std::sqrt(2.0 / (double)fan_in);
        unwrap(rh_rng_fill_normal(seed[0], seed[1], w.data(), wlen, 0.0f, sd), "rh_rng_fill_normal");
        break;
      }
    }
    std::vector<float> b(blen, 0.0f);
    weights->sync_load(w.data(), wlen);
    bias->sync_load(b.data(), blen);
  }
  void encode_pair(std::vector<uint8_t>& blob, const DeviceBuffer<float>& w, const DeviceBuffer<float>& b) const {
    ctx->sync();
    std::vector<float> hw(wlen), hb(blen);
    w.sync_store(hw.data(), wlen);
    b.sync_store(hb.data(), blen);
    const size_t wd[2] = {wrows, wcols}, bd[2] = {1, blen};
    ndarray_serialize(blob, hw.data(), wd, 2);
    ndarray_serialize(blob, hb.data(), bd, 2);
  }
  size_t decode_pair(const uint8_t* blob, size_t len, DeviceBuffer<float>& w, DeviceBuffer<float>& b, const char* who) {
    std::vector<size_t> dims;
    std::vector<float> data;
    size_t off = ndarray_deserialize(blob, len, &dims, &data);
    if (dims.size() != 2 || dims[0] != wrows || dims[1] != wcols) panic(std::string(who) + ": weights blob has the wrong bound");
    w.sync_load(data.data(), wlen);
    off += ndarray_deserialize(blob + off, len - off, &dims, &data);
    if (dims.size() != 2 || dims[0] != 1 || dims[1] != blen) panic(std::string(who) + ": bias blob has the wrong bound");
    b.sync_load(data.data(), blen);
    return off;
  }
  void encode_params(std::vector<uint8_t>& blob) const { encode_pair(blob, *weights, *bias); }
  size_t decode_params(const uint8_t* blob, size_t len, const char* who) { return decode_pair(blob, len, *weights, *bias, who); }
  void encode_state(std::vector<uint8_t>& blob) const {
    RB_ASSERT(has_backward());
    encode_pair(blob, *acc_grad_weights, *acc_grad_bias);
  }
  size_t decode_state(const uint8_t* blob, size_t len, const char* who) {
    RB_ASSERT(has_backward());
    return decode_pair(blob, len, *acc_grad_weights, *acc_grad_bias, who);
  }
  bool buffer(int which, float** ptr, size_t* len) {
    DeviceBuffer<float>* b = nullptr;
    if ((which == 4 || which == 5) && has_backward()) touch_grads();
    switch (which) {
      case 2: b = weights.get(); break;
      case 3: b = bias.get(); break;
      case 4: b = grad_weights.get(); break;
      case 5: b = grad_bias.get(); break;
      case 6: b = acc_grad_weights.get(); break;
      case 7: b = acc_grad_bias.get(); break;
      default: return false;
    }
    if (!b) return false;
    *ptr = b->as_mut_ptr();
    *len = b->len();
    return true;
  }
};

void apply_rect(ActivationFunction f, float* y, size_t frame_len, size_t batch, rh_stream_t s) {
  switch (f) {
    case ActivationFunction::Identity: break;
    case ActivationFunction::Rect:
      rembrandt_kernel_batch_map_rect_inplace(y, (int32_t)frame_len, (int32_t)batch, s);
      unwrap_last("rembrandt_kernel_batch_map_rect_inplace");
      break;
    default: panic("unimplemented activation function");
  }
}

void apply_rect_backprop(ActivationFunction f, const float* y, size_t frame_len, size_t batch, float* dy, rh_stream_t s) {
  switch (f) {
    case ActivationFunction::Identity: break;
    case ActivationFunction::Rect:
      rembrandt_kernel_batch_map_rect_backprop_inplace(y, (int32_t)frame_len, (int32_t)batch, dy, s);
      unwrap_last("rembrandt_kernel_batch_map_rect_backprop_inplace");
      break;
    default: panic("unimplemented activation function");
  }
}

// xorshift128+ for per-operator seed derivation (Xorshiftplus128Rng in src/operator/worker.rs:361-367) and the
// input operator's crop / flip draws (src/operator/mod.rs:503,619); the reference's bit streams are not reproducible here.
struct Xorshiftplus128 {
  uint64_t s0, s1;
  explicit Xorshiftplus128(const uint64_t seed[2]) : s0(seed[0]), s1(seed[1]) {
    if (s0 == 0 && s1 == 0) s1 = 0x9E3779B97F4A7C15ull;
  }
  uint64_t next_u64() {
    uint64_t x = s0;
    const uint64_t y = s1;
    s0 = y;
    x ^= x << 23;
    s1 = x ^ y ^ (x >> 17) ^ (y >> 26);
    return s1 + y;
  }
};


// ---- Data3dOperator ---------------------------------------------------------------------------------------
// u8 staging -> H2D -> cast (optionally /255) -> preprocessing steps ping-ponging between tmp_buf and out_buf so
// that the last one lands in out_buf (src/operator/mod.rs:640-790).  Crop offsets and the flip coin are drawn
// once per forward() for the whole batch, as in the reference; Inference uses the centre crop and no flip/noise.
class Data3dOperator : public InputOperator {
 public:
  Data3dOperator(size_t batch_size, const Data3dOperatorConfig& config, Ctx context, const uint64_t seed[2])
      : batch_cap_(batch_size), config_(config), context_(context),
        in_buf_h_(batch_size * config.in_dims.len(), context),
        in_buf_(new DeviceBuffer<uint8_t>(batch_size * config.in_dims.len(), context)),
        out_buf_(new DeviceBuffer<float>(batch_size * config.in_dims.len(), context)),
        rng_(seed), noise_seed_(seed[0] ^ 0x5043414Eull) {
    (void)config_.get_out_dims();  // asserts that every crop fits
    if (!config.preprocs.empty()) tmp_buf_.reset(new DeviceBuffer<float>(batch_size * config.in_dims.len(), context));
    for (const auto& p : config.preprocs) {
      PreprocState st;
      if (p.kind == Data3dPreproc::SubtractElemwiseMean) {
        std::vector<float> mean = p.mean_values;
        if (!p.mean_path.empty()) {
          std::ifstream f(p.mean_path, std::ios::binary);
          if (!f) panic("failed to open mean path: " + p.mean_path);
          std::vector<uint8_t> blob((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
          std::vector<size_t> dims;
          ndarray_deserialize(blob.data(), blob.size(), &dims, &mean);
        }
        if (mean.size() != config.in_dims.len()) panic("failed to deserialize mean array: wrong length");
        st.dev.reset(new DeviceBuffer<float>(mean.size(), context));
        st.dev->sync_load(mean.data(), mean.size());
      } else if (p.kind == Data3dPreproc::AddPixelwisePCALightingNoise) {
        RB_ASSERT(config.in_dims.c == 3);
        // [svecs: 9][svals: 3][alphas: 3*batch]
        st.dev.reset(new DeviceBuffer<float>(12 + 3 * batch_size, context));
        float h[12];
        for (int i = 0; i < 3; ++i)
          for (int j = 0; j < 3; ++j) h[i * 3 + j] = p.singular_vecs[i][j];
        for (int j = 0; j < 3; ++j) h[9 + j] = p.singular_vals[j];
        st.dev->sync_load(h, 12);
      }
      states_.push_back(std::move(st));
    }
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_buf_; }
  SharedDeviceBuf get_output_deltas() const override { return nullptr; }  // src/operator/mod.rs:632-634
  Dims3 out_dims() const override { return config_.get_out_dims(); }
  size_t in_frame_len() const override { return config_.in_dims.len(); }
  uint8_t* expose_host_frame_buf(size_t batch_idx) override {
    RB_ASSERT(batch_idx < batch_cap_);
    return in_buf_h_.data() + batch_idx * config_.in_dims.len();
  }
  // The copy runs on the context's copy stream, beside whatever the main stream still holds of the previous batch
  // (its backward pass and update), and only after that batch's cast has read in_buf; forward() marks that point.
  void load_frames(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    unwrap(rh_load_overlapped(context_->raw(), in_buf_->as_mut_ptr(), in_buf_h_.data(), in_buf_h_.size()), "sync_load");
    f32_loaded_ = false;
  }
  void load_frames_f32(const float* host, size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const size_t n = batch_size * config_.in_dims.len();
    if (config_.preprocs.empty()) {
      out_buf_->sync_load(host, n);  // frames are placed where the cast would put them
    } else {
      if (!f32_frames_) f32_frames_.reset(new DeviceBuffer<float>(batch_cap_ * config_.in_dims.len(), context_));
      f32_frames_->sync_load(host, n);
    }
    f32_loaded_ = true;
  }
  void forward(size_t batch_size, OpPhase phase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    rh_stream_t s = context_->stream();
    const size_t num_preprocs = config_.preprocs.size();
    const size_t in_len = batch_size * config_.in_dims.len();
    float* const out = out_buf_->as_mut_ptr();
    float* const tmp = tmp_buf_ ? tmp_buf_->as_mut_ptr() : nullptr;
    float* cur = num_preprocs % 2 == 0 ? out : tmp;
    if (f32_loaded_) {
      if (num_preprocs) unwrap(rh_copy_d2d(cur, f32_frames_->as_ptr(), in_len * sizeof(float), s), "send");
    } else {
      unwrap(rh_cast_u8_f32(in_buf_->as_ptr(), cur, in_len, config_.normalize ? 1.0f / 255.0f : 1.0f, s), "cast_bytes");
      unwrap(rh_mark_consumed(context_->raw()), "mark_consumed");  // in_buf may be refilled from here on
    }
    Dims3 dims = config_.in_dims;
    last_alphas_.clear();
    last_flip_ = false;
    for (size_t r = 0; r < num_preprocs; ++r) {
      const Data3dPreproc& p = config_.preprocs[r];
      float* const dst = cur == out ? tmp : out;
      const size_t len = batch_size * dims.len();
      switch (p.kind) {
        case Data3dPreproc::Crop: {
          size_t off_w, off_h;
          if (phase.training) {  // uniform over [0, max_offset] (src/operator/mod.rs:553-569, 681-685)
            off_w = (size_t)(rng_.next_u64() % (uint64_t)(dims.w - p.crop_width + 1));
            off_h = (size_t)(rng_.next_u64() % (uint64_t)(dims.h - p.crop_height + 1));
          } else {
            off_w = (dims.w - p.crop_width) / 2;
            off_h = (dims.h - p.crop_height) / 2;
          }
          last_off_w_ = off_w;
          last_off_h_ = off_h;
          unwrap(rh_crop_nchw(cur, dst, (int64_t)(batch_size * dims.c), (int)dims.w, (int)dims.h, (int)p.crop_width,
                              (int)p.crop_height, (int)off_w, (int)off_h, s), "crop transform");
          dims = {p.crop_width, p.crop_height, dims.c};
          break;
        }
        case Data3dPreproc::FlipX: {
          const bool flip = phase.training && (rng_.next_u64() & 1);
          last_flip_ = flip;
          if (flip) {
            rembrandt_kernel_batch_blockmap256_flip(cur, (int32_t)dims.w, (int32_t)(dims.h * dims.c * batch_size), dst, s);
            unwrap_last("rembrandt_kernel_batch_blockmap256_flip");
          } else {
            unwrap(rh_copy_d2d(dst, cur, len * sizeof(float), s), "send");
          }
          break;
        }
        case Data3dPreproc::SubtractElemwiseMean: {
          RB_ASSERT(dims.len() == config_.in_dims.len());  // the mean has the input frame's shape
          const float alpha = config_.normalize ? -1.0f / 255.0f : -1.0f;
          unwrap(rh_copy_d2d(dst, cur, len * sizeof(float), s), "send");
          unwrap(rh_add_bias_nchw(states_[r].dev->as_ptr(), dst, 1, (int32_t)dims.len(), (int32_t)batch_size, alpha, 1.0f, s),
                 "subtract mean");
          break;
        }
        case Data3dPreproc::AddPixelwisePCALightingNoise: {
          if (phase.training) {
            last_alphas_.resize(3 * batch_size);
            unwrap(rh_rng_fill_normal(noise_seed_, noise_draws_++, last_alphas_.data(), last_alphas_.size(), 0.0f, p.std_dev),
                   "sample alphas");
            float* base = states_[r].dev->as_mut_ptr();
            unwrap(rh_load_sync(context_->raw(), base + 12, last_alphas_.data(), last_alphas_.size() * sizeof(float)), "sync_load");
            rembrandt_kernel_batch_map_preproc_pca3_noise(cur, (int32_t)(dims.w * dims.h), (int32_t)batch_size, base + 12,
                                                          base + 9, base, dst, s);
            unwrap_last("rembrandt_kernel_batch_map_preproc_pca3_noise");
          } else {
            unwrap(rh_copy_d2d(dst, cur, len * sizeof(float), s), "send");
          }
          break;
        }
      }
      cur = dst;
    }
  }
  void backward(size_t) override {}
  void last_preproc_draws(size_t* crop_off_w, size_t* crop_off_h, bool* flipped, std::vector<float>* alphas) const override {
    if (crop_off_w) *crop_off_w = last_off_w_;
    if (crop_off_h) *crop_off_h = last_off_h_;
    if (flipped) *flipped = last_flip_;
    if (alphas) *alphas = last_alphas_;
  }
  int input_mode() const override { return f32_loaded_ ? 1 : 0; }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which != 0) return false;
    *ptr = out_buf_->as_mut_ptr();
    *len = out_buf_->len();
    return true;
  }
  const char* kind() const override { return "Data3dOperator"; }
  // random crops, flips and lighting noise draw new launch arguments for every training batch
  bool graph_safe(OpPhase phase) const override {
    if (!phase.training) return true;
    for (const auto& p : config_.preprocs)
      if (p.kind != Data3dPreproc::SubtractElemwiseMean) return false;
    return true;
  }

 private:
  struct PreprocState {
    std::unique_ptr<DeviceBuffer<float>> dev;
  };
  size_t batch_cap_;
  Data3dOperatorConfig config_;
  Ctx context_;
  PinnedBytes in_buf_h_;  // page-locked: it is copied to the device every batch
  std::unique_ptr<DeviceBuffer<uint8_t>> in_buf_;
  std::unique_ptr<DeviceBuffer<float>> tmp_buf_, f32_frames_;
  SharedDeviceBuf out_buf_;
  std::vector<PreprocState> states_;
  Xorshiftplus128 rng_;
  uint64_t noise_seed_, noise_draws_ = 0;
  size_t last_off_w_ = 0, last_off_h_ = 0;
  bool last_flip_ = false;
  std::vector<float> last_alphas_;
  bool f32_loaded_ = false;
};

// ---- AffineOperator -------------------------------------------------------------------------------------
class AffineOperator : public Operator {
 public:
  AffineOperator(size_t batch_size, OpCapability capability, const AffineOperatorConfig& config, const Operator* prev_op,
                 Ctx context, const ExecOptions& opts)
      : batch_cap_(batch_size), config_(config), context_(context), fuse_epilogue_(opts.fuse_epilogue),
        overlap_built_(opts.overlap_backward && backward_enabled(capability)), overlap_on_(overlap_built_) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("AffineOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.in_channels * batch_size);
    out_act_.reset(new DeviceBuffer<float>(config.out_channels * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(config.out_channels * batch_size, context));
    params_.alloc(config.in_channels * config.out_channels, config.out_channels, backward_enabled(capability), context);
    const int i = (int)config.in_channels, o = (int)config.out_channels, b = (int)batch_size;
    size_t ws = sgemm_ws_upto(o, b, i, 1, b);
    if (backward_enabled(capability)) {
      ws = std::max(ws, sgemm_ws_upto(i, o, b, 2, b));
      ws = std::max(ws, sgemm_ws_upto(i, b, o, 1, b));
    }
    if (ws) workspace_.reset(new DeviceBuffer<uint8_t>(ws, context));
    if (overlap_built_) {
      const size_t wa = sgemm_ws_upto(i, o, b, 2, b);
      if (wa) workspace_aux_.reset(new DeviceBuffer<uint8_t>(wa, context));
    }
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void init_params(const uint64_t seed[2]) override {
    params_.init(config_.init_weights, seed, config_.in_channels, config_.out_channels, true, "AffineOperator");
  }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const int i = (int)config_.in_channels, o = (int)config_.out_channels, b = (int)batch_size;
    rh_stream_t s = context_->stream();
    // out_act(out, B) = weights(in, out)^T * in_act(in, B)
    const bool rect = config_.act_func == ActivationFunction::Rect;
    if (fuse_epilogue_ && (rect || config_.act_func == ActivationFunction::Identity)) {
      // bias and activation in the product's epilogue: one kernel for the reference's three
      unwrap(rh_sgemm_bias_act(1, 0, o, b, i, 1.0f, params_.weights->as_ptr(), i, in_act_->as_ptr(), i, 0.0f,
                               out_act_->as_mut_ptr(), o, params_.bias->as_ptr(), ws_ptr(), ws_len(),
                               RH_FUSE_BIAS | (rect ? RH_FUSE_RELU : 0), s), "matrix_prod");
      return;
    }
    unwrap(rh_sgemm(1, 0, o, b, i, 1.0f, params_.weights->as_ptr(), i, in_act_->as_ptr(), i, 0.0f,
                    out_act_->as_mut_ptr(), o, ws_ptr(), ws_len(), 0, s), "matrix_prod");
    unwrap(rh_add_bias_nchw(params_.bias->as_ptr(), out_act_->as_mut_ptr(), 1, o, b, 1.0f, 1.0f, s), "add_bias");
    apply_rect(config_.act_func, out_act_->as_mut_ptr(), config_.out_channels, batch_size, s);
  }
  void backward(size_t batch_size) override {
    RB_ASSERT(params_.has_backward());
    RB_ASSERT(batch_size <= batch_cap_);
    const int i = (int)config_.in_channels, o = (int)config_.out_channels, b = (int)batch_size;
    rh_stream_t s = context_->stream();
    if (!delta_masked_once_)
      apply_rect_backprop(config_.act_func, out_act_->as_ptr(), config_.out_channels, batch_size, out_delta_->as_mut_ptr(), s);
    delta_masked_once_ = false;
    // The two parameter gradients go to the second stream when a data gradient follows on the main stream (scratch
    // of their own there); the worker joins at the end of backward.
    rh_stream_t sg = s;
    void* wg = ws_ptr();
    size_t wg_len = ws_len();
    if (overlap_on_ && in_delta_) {
      context_->fork();
      sg = context_->aux_stream();
      wg = workspace_aux_ ? workspace_aux_->as_mut_ptr() : nullptr;
      wg_len = workspace_aux_ ? workspace_aux_->len() : 0;
    }
    const float beta = params_.take_backward_beta();   // 1: accumulate (the reference's call); 0: the buffers stand for zeros
    // grad_weights(in, out) += in_act(in, B) * out_delta(out, B)^T
    unwrap(rh_sgemm(0, 1, i, o, b, 1.0f, in_act_->as_ptr(), i, out_delta_->as_ptr(), o, beta,
                    params_.grad_weights->as_mut_ptr(), i, wg, wg_len, 0, sg), "matrix_prod");
    // grad_bias(1, out) += 1(1, B) * out_delta^T: the column sums of out_delta, without the ones vector
    if (!bias_grad_done_)
      unwrap(rh_conv2d_bwd_bias(b, o, 1, 1.0f, out_delta_->as_ptr(), beta, params_.grad_bias->as_mut_ptr(), sg), "matrix_prod");
    bias_grad_done_ = false;
    if (in_delta_) {
      // in_delta(in, B) = weights(in, out) * out_delta(out, B)
      unwrap(rh_sgemm(0, 0, i, b, o, 1.0f, params_.weights->as_ptr(), i, out_delta_->as_ptr(), o, 0.0f,
                      in_delta_->as_mut_ptr(), i, ws_ptr(), ws_len(), 0, s), "matrix_prod");
    }
  }
  void regularize(Regularization reg) override { params_.regularize(reg); }
  void accumulate_grads(float scale, float momentum) override { params_.accumulate_grads(scale, momentum); }
  void update_params(float scale) override { params_.update_params(scale); }
  void update_params2(float g, float u) override { params_.update_params2(g, u); }
  void save_params() override { params_.save_params(); }
  void restore_params() override { params_.restore_params(); }
  void reset() override { params_.reset(); }
  // backward_scaled: the inherited form; AffineLayer::backward accumulates both gradients with factor 1.0 whatever
  // `scale` is (src/layer_new.rs:583-584)
  void descend(float scale, float l2, bool fused) override { params_.descend(scale, l2, fused); }
  void reset_gradients(float scale) override { params_.reset_gradients(scale); }
  void encode_params(std::vector<uint8_t>& blob) override { params_.encode_params(blob); }
  size_t decode_params(const uint8_t* blob, size_t len) override { return params_.decode_params(blob, len, kind()); }
  void encode_state(std::vector<uint8_t>& blob) override { params_.encode_state(blob); }
  size_t decode_state(const uint8_t* blob, size_t len) override { return params_.decode_state(blob, len, kind()); }
  void fused_sgd_step(float l2, float scale, float mu, float apply) override {
    params_.fused_sgd_step(l2, scale, mu, apply, overlap_on_ ? context_->aux_stream() : nullptr);
  }
  void sgd_tensors(float l2, std::vector<rh_sgd_tensor>& out) override { params_.sgd_tensors(l2, out); }
  bool grads_stale() const override { return params_.grads_stale; }
  void set_grads_stale(bool stale) override { params_.grads_stale = stale && params_.has_backward(); }
  bool updates_on_second_stream() const override { return overlap_on_; }
  void set_overlap_backward(bool on) override { overlap_on_ = on && overlap_built_; }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    return params_.buffer(which, ptr, len);
  }
  const char* kind() const override { return "AffineOperator"; }

 private:
  friend struct ::rembrandt::ClassifierTail;
  void* ws_ptr() { return workspace_ ? workspace_->as_mut_ptr() : nullptr; }
  size_t ws_len() { return workspace_ ? workspace_->len() : 0; }
  size_t batch_cap_;
  AffineOperatorConfig config_;
  Ctx context_;
  bool fuse_epilogue_;               // bias and activation inside the forward product
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  ParamTensors params_;
  std::unique_ptr<DeviceBuffer<uint8_t>> workspace_, workspace_aux_;
  bool overlap_built_, overlap_on_;  // parameter gradients and the fused SGD step of this block on the second stream
  bool delta_masked_once_ = false;   // out_delta_ already went through the activation's backward (the classifier tail)
  bool bias_grad_done_ = false;      // this pass's bias gradient is already in grad_bias (the classifier tail's launch formed it)
};

// ---- Conv2dOperator -------------------------------------------------------------------------------------
class Conv2dOperator : public Operator {
 public:
  Conv2dOperator(size_t batch_size, OpCapability capability, const Conv2dOperatorConfig& config, Operator* prev_op,
                 Ctx context, ExecOptions opts)
      : batch_cap_(batch_size), config_(config), context_(context), opts_(opts) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("Conv2dOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    out_dims_ = config.get_out_dims();
    out_act_.reset(new DeviceBuffer<float>(out_dims_.len() * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(out_dims_.len() * batch_size, context));
    params_.alloc(config.conv_size * config.conv_size * config.in_dims.c * config.out_channels, config.out_channels,
                  backward_enabled(capability), context);
    // one scratch buffer sized for the largest of the three passes (src/operator/mod.rs:1493-1507)
    const rh_conv_geom g = geom(batch_size);
    size_t ws = conv_ws_upto(g, RH_CONV_FWD);
    if (backward_enabled(capability)) {
      ws = std::max(ws, conv_ws_upto(g, RH_CONV_BWD_FILTER));
      ws = std::max(ws, conv_ws_upto(g, RH_CONV_BWD_DATA));
      ws = std::max(ws, bias_ws_upto(g.N, g.K, (int)(out_dims_.w * out_dims_.h)));
    }
    workspace_.reset(new DeviceBuffer<uint8_t>(std::max<size_t>(ws, 256), context));
    if (backward_enabled(capability) && opts.overlap_backward) {
      // the filter / bias gradients run on the second stream with scratch of their own
      size_t wa = conv_ws_upto(g, RH_CONV_BWD_FILTER);
      wa = std::max(wa, bias_ws_upto(g.N, g.K, (int)(out_dims_.w * out_dims_.h)));
      workspace_aux_.reset(new DeviceBuffer<uint8_t>(std::max<size_t>(wa, 256), context));
    }
    // the data gradient can zero what the ReLU below would have masked in a pass of its own
    if (backward_enabled(capability) && in_delta_ && opts.fuse_epilogue && rh_conv2d_bwd_data_relu_supported(&g))
      fold_prev_relu_ = prev_op->fold_activation_backward();
    if (opts.bf16_forward) {
      // the converted filter is kept from one forward pass to the next for as long as the weights stay the same
      const size_t fb = rh_conv2d_fwd_bf16_filter_bytes(&g);
      if (fb) {
        wprep_.reset(new DeviceBuffer<uint8_t>(fb, context));
        const size_t wb = rh_conv2d_fwd_bf16_workspace_bytes(&g);
        if (wb > workspace_->len()) workspace_.reset(new DeviceBuffer<uint8_t>(wb, context));
        if (opts.bf16_packed_chain && rh_conv2d_fwd_bf16_takes_packed(&g) && prev_op->can_emit_packed())
          in_packed_ = prev_op->emit_packed(g.pad);
      }
    }
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void init_params(const uint64_t seed[2]) override {
    const size_t fan_in = config_.conv_size * config_.conv_size * config_.in_dims.c;
    params_.init(config_.init_weights, seed, fan_in, config_.out_channels, false, "Conv2dOperator");
    wprep_valid_ = false;
  }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_conv_geom g = geom(batch_size);
    rh_stream_t s = context_->stream();
    const bool rect = config_.act_func == ActivationFunction::Rect;
    if (config_.act_func != ActivationFunction::Identity && !rect) panic("unimplemented activation function");
    if (wprep_) {
      if (!wprep_valid_) {
        unwrap(rh_conv2d_fwd_bf16_prep_filter(&g, params_.weights->as_ptr(), wprep_->as_mut_ptr(), wprep_->len(), s),
               "conv2d forward (filter conversion)");
        wprep_valid_ = true;
      }
      const int flags = opts_.fuse_epilogue ? RH_FUSE_BIAS | (rect ? RH_FUSE_RELU : 0) : 0;
      unwrap(rh_conv2d_fwd_bf16_packed(&g, in_packed_ ? in_packed_->as_ptr() : nullptr, in_packed_ ? nullptr : in_act_->as_ptr(),
                                       wprep_->as_ptr(), params_.bias->as_ptr(), out_packed_ ? nullptr : out_act_->as_mut_ptr(),
                                       out_packed_ ? out_packed_->as_mut_ptr() : nullptr, out_halo_, workspace_->as_mut_ptr(),
                                       workspace_->len(), flags, s), "conv2d forward");
      if (!opts_.fuse_epilogue) {   // (never with a packed output: can_emit_packed asks for the fused epilogue)
        unwrap(rh_add_bias_nchw(params_.bias->as_ptr(), out_act_->as_mut_ptr(), (int)(out_dims_.w * out_dims_.h),
                                (int)out_dims_.c, (int)batch_size, 1.0f, 1.0f, s), "add_bias");
        apply_rect(config_.act_func, out_act_->as_mut_ptr(), out_dims_.len(), batch_size, s);
      }
      return;
    }
    const int math = (opts_.bf16_forward ? RH_MATH_BF16_MFMA_FP32ACC : 0) | (opts_.winograd ? 0 : RH_ALGO_DIRECT);
    if (opts_.fuse_epilogue) {
      const int flags = RH_FUSE_BIAS | (rect ? RH_FUSE_RELU : 0) | math;
      unwrap(rh_conv2d_fwd(&g, 1.0f, in_act_->as_ptr(), params_.weights->as_ptr(), 0.0f, out_act_->as_mut_ptr(),
                           params_.bias->as_ptr(), workspace_->as_mut_ptr(), workspace_->len(), flags, s), "conv2d forward");
    } else {
      unwrap(rh_conv2d_fwd(&g, 1.0f, in_act_->as_ptr(), params_.weights->as_ptr(), 0.0f, out_act_->as_mut_ptr(), nullptr,
                           workspace_->as_mut_ptr(), workspace_->len(), math, s), "conv2d forward");
      unwrap(rh_add_bias_nchw(params_.bias->as_ptr(), out_act_->as_mut_ptr(), (int)(out_dims_.w * out_dims_.h),
                              (int)out_dims_.c, (int)batch_size, 1.0f, 1.0f, s), "add_bias");
      apply_rect(config_.act_func, out_act_->as_mut_ptr(), out_dims_.len(), batch_size, s);
    }
  }
  void backward(size_t batch_size) override { backward_scaled(batch_size, 1.0f); }
  // `scale` is the factor of the filter and bias gradients (the alpha of backward_filter / backward_bias,
  // src/layer_new.rs:1093-1108); the operator generation always passes 1 (src/operator/mod.rs:1765-1781).
  void backward_scaled(size_t batch_size, float scale) override {
    RB_ASSERT(params_.has_backward());
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_conv_geom g = geom(batch_size);
    rh_stream_t s = context_->stream();
    if (!act_bwd_folded_)
      apply_rect_backprop(config_.act_func, out_act_->as_ptr(), out_dims_.len(), batch_size, out_delta_->as_mut_ptr(), s);
    // Streams and scratch of the two gradient kernels.  With a data gradient to follow on the main stream both go
    // to the second stream; the first layer has none, so its gradients stay on the main stream (on the second
    // they would only queue behind that stream's earlier work).
    rh_stream_t s_filter = s, s_bias = s;
    DeviceBuffer<uint8_t>*w_filter = workspace_.get(), *w_bias = workspace_.get();
    if (workspace_aux_ && overlap_on_ && in_delta_) {
      context_->fork();                        // the second stream sees the masked out_delta
      s_filter = s_bias = context_->aux_stream();
      w_filter = w_bias = workspace_aux_.get();
    }
    const float beta = params_.take_backward_beta();   // 1: accumulate (the reference's call); 0: the buffers stand for zeros
    const int algo = opts_.winograd ? 0 : RH_ALGO_DIRECT;
    // (a small layer's bias gradient rides in the launch of the filter gradient's reduction: the combined call below)
    const bool small = batch_size * out_dims_.len() <= (size_t(1) << 20);
    if (!in_delta_ && workspace_aux_ && overlap_on_ && !small) {
      // First layer, backward on two streams: its gradients are the last kernels of the pass.  The bias gradient goes
      // first (a memory-bound pass beside the second stream's last contraction), so that only the filter gradient's
      // reduction follows the last contraction of the step.
      unwrap(rh_conv2d_bwd_bias_ws((int)batch_size, (int)out_dims_.c, (int)(out_dims_.w * out_dims_.h), scale,
                                   out_delta_->as_ptr(), beta, params_.grad_bias->as_mut_ptr(), w_bias->as_mut_ptr(),
                                   w_bias->len(), s_bias), "conv2d backward bias");
      unwrap(rh_conv2d_bwd_filter(&g, scale, in_act_->as_ptr(), out_delta_->as_ptr(), beta, params_.grad_weights->as_mut_ptr(),
                                  w_filter->as_mut_ptr(), w_filter->len(), algo, s_filter), "conv2d backward filter");
    } else if (s_filter == s_bias && w_filter == w_bias) {
      // one stream for both: one call, which reads out_delta once where the filter gradient makes a pass over it anyway
      unwrap(rh_conv2d_bwd_filter_bias(&g, scale, in_act_->as_ptr(), out_delta_->as_ptr(), beta,
                                       params_.grad_weights->as_mut_ptr(), params_.grad_bias->as_mut_ptr(),
                                       w_filter->as_mut_ptr(), w_filter->len(), algo, s_filter), "conv2d backward filter / bias");
    } else {
      unwrap(rh_conv2d_bwd_filter(&g, scale, in_act_->as_ptr(), out_delta_->as_ptr(), beta, params_.grad_weights->as_mut_ptr(),
                                  w_filter->as_mut_ptr(), w_filter->len(), algo, s_filter), "conv2d backward filter");
      unwrap(rh_conv2d_bwd_bias_ws((int)batch_size, (int)out_dims_.c, (int)(out_dims_.w * out_dims_.h), scale,
                                   out_delta_->as_ptr(), beta, params_.grad_bias->as_mut_ptr(), w_bias->as_mut_ptr(),
                                   w_bias->len(), s_bias), "conv2d backward bias");
    }
    const int beside = s_filter != s ? RH_ALGO_SHARED_GPU : 0;   // the filter gradient runs beside the data gradient
    if (in_delta_ && fold_prev_relu_) {
      // the operator below left its ReLU backward mask to this call: in_act_ is that ReLU's output
      unwrap(rh_conv2d_bwd_data_relu(&g, 1.0f, params_.weights->as_ptr(), out_delta_->as_ptr(), 0.0f, in_delta_->as_mut_ptr(),
                                     in_act_->as_ptr(), workspace_->as_mut_ptr(), workspace_->len(), algo | beside, s),
             "conv2d backward data");
    } else if (in_delta_) {
      unwrap(rh_conv2d_bwd_data(&g, 1.0f, params_.weights->as_ptr(), out_delta_->as_ptr(), 0.0f, in_delta_->as_mut_ptr(),
                                workspace_->as_mut_ptr(), workspace_->len(), algo | beside, s),
             "conv2d backward data");
    }
  }
  void regularize(Regularization reg) override { params_.regularize(reg); }
  void accumulate_grads(float scale, float momentum) override { params_.accumulate_grads(scale, momentum); }
  // (every method that can change the weights drops the converted filter of the bf16 forward)
  void update_params(float scale) override { wprep_valid_ = false; params_.update_params(scale); }
  void update_params2(float g, float u) override { wprep_valid_ = false; params_.update_params2(g, u); }
  void save_params() override { params_.save_params(); }
  void restore_params() override { wprep_valid_ = false; params_.restore_params(); }
  void reset() override { params_.reset(); }
  void descend(float scale, float l2, bool fused) override { wprep_valid_ = false; params_.descend(scale, l2, fused); }
  void reset_gradients(float scale) override { params_.reset_gradients(scale); }
  void encode_params(std::vector<uint8_t>& blob) override { params_.encode_params(blob); }
  size_t decode_params(const uint8_t* blob, size_t len) override {
    wprep_valid_ = false;
    return params_.decode_params(blob, len, kind());
  }
  void encode_state(std::vector<uint8_t>& blob) override { params_.encode_state(blob); }
  size_t decode_state(const uint8_t* blob, size_t len) override { return params_.decode_state(blob, len, kind()); }
  // Like the affine layers' updates, on the second stream, except for the first layer: the next forward pass joins
  // in front of the first operator that was updated there, and the first layer's forward is what the others hide behind.
  void fused_sgd_step(float l2, float scale, float mu, float apply) override {
    wprep_valid_ = false;
    params_.fused_sgd_step(l2, scale, mu, apply, updates_on_second_stream() ? context_->aux_stream() : nullptr);
  }
  void sgd_tensors(float l2, std::vector<rh_sgd_tensor>& out) override { wprep_valid_ = false; params_.sgd_tensors(l2, out); }
  bool grads_stale() const override { return params_.grads_stale; }
  void set_grads_stale(bool stale) override { params_.grads_stale = stale && params_.has_backward(); }
  bool updates_on_second_stream() const override { return workspace_aux_ && overlap_on_ && in_delta_; }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) {
      if (out_packed_)   // the activations live in the packed buffer: their values as fp32, on demand
        unwrap(rh_bf16_unpack_nchw((int)batch_cap_, (int)out_dims_.c, (int)out_dims_.h, (int)out_dims_.w, out_halo_,
                                   out_packed_->as_ptr(), out_act_->as_mut_ptr(), context_->stream()), "bf16 unpack");
      *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true;
    }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    if (which == 2 || which == 3) wprep_valid_ = false;   // the caller may write through the pointer
    return params_.buffer(which, ptr, len);
  }
  bool can_emit_packed() const override {
    return opts_.bf16_packed_chain && opts_.fuse_epilogue && wprep_ && !out_packed_ && out_dims_.c % 8 == 0 &&
           rh_bf16_act_bytes((int)batch_cap_, (int)out_dims_.c, (int)out_dims_.h, (int)out_dims_.w, 0) > 0;
  }
  std::shared_ptr<DeviceBuffer<uint8_t>> emit_packed(int halo) override {
    const size_t bytes = rh_bf16_act_bytes((int)batch_cap_, (int)out_dims_.c, (int)out_dims_.h, (int)out_dims_.w, halo);
    if (!can_emit_packed() || !bytes) panic("Conv2dOperator: no packed output for this configuration");
    out_packed_.reset(new DeviceBuffer<uint8_t>(bytes, context_));   // zero-filled: the border stays zero
    out_halo_ = halo;
    return out_packed_;
  }
  const char* kind() const override { return "Conv2dOperator"; }
  bool fold_activation_backward() override {
    if (config_.act_func != ActivationFunction::Rect) return false;
    act_bwd_folded_ = true;
    return true;
  }
  void set_overlap_backward(bool on) override { overlap_on_ = on; }

 private:
  bool act_bwd_folded_ = false;   // the operator above applies this operator's ReLU backward mask
  bool fold_prev_relu_ = false;   // this operator's data gradient applies the ReLU backward mask of the operator below
  rh_conv_geom geom(size_t batch) const {
    rh_conv_geom g;
    g.N = (int)batch; g.C = (int)config_.in_dims.c; g.H = (int)config_.in_dims.h; g.W = (int)config_.in_dims.w;
    g.K = (int)config_.out_channels; g.R = g.S = (int)config_.conv_size;
    g.stride = (int)config_.conv_stride; g.pad = (int)config_.conv_pad;
    return g;
  }
  size_t batch_cap_;
  Conv2dOperatorConfig config_;
  Ctx context_;
  ExecOptions opts_;
  Dims3 out_dims_;
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  ParamTensors params_;
  std::unique_ptr<DeviceBuffer<uint8_t>> workspace_, workspace_aux_;
  bool overlap_on_ = true;
  // bf16 forward: the converted filter (valid until the weights change) and the packed activations on either side
  std::unique_ptr<DeviceBuffer<uint8_t>> wprep_;
  bool wprep_valid_ = false;
  std::shared_ptr<DeviceBuffer<uint8_t>> in_packed_, out_packed_;
  int out_halo_ = 0;
};

// ---- Pool2dOperator -------------------------------------------------------------------------------------
class Pool2dOperator : public Operator {
 public:
  Pool2dOperator(size_t batch_size, const Pool2dOperatorConfig& config, Operator* prev_op, Ctx context, const ExecOptions& opts)
      : batch_cap_(batch_size), config_(config), context_(context), prev_op_(prev_op),
        packed_chain_(opts.bf16_packed_chain) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("Pool2dOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    out_dims_ = config.get_out_dims();
    out_act_.reset(new DeviceBuffer<float>(out_dims_.len() * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(out_dims_.len() * batch_size, context));
    // private arg-max mask: lets backward route deltas without re-scanning the windows
    if (config.pool_op == PoolOperation::Max && in_delta_) {
      const rh_pool_geom g = geom(batch_size);
      // one byte per window (the winner's slot) where the library has that form, else the int32 plane index
      if (rh_pool2d_slot_supported(&g)) slot_.reset(new DeviceBuffer<uint8_t>(out_dims_.len() * batch_size, context));
      else argmax_.reset(new DeviceBuffer<int32_t>(out_dims_.len() * batch_size, context));
      if (opts.fuse_epilogue && rh_pool2d_bwd_relu_supported(&g)) fold_relu_ = prev_op->fold_activation_backward();
    }
    // average pooling: the same fold, with the pool's input (the ReLU's output) as the mask
    if (config.pool_op == PoolOperation::Average && in_delta_ && opts.fuse_epilogue)
      fold_relu_ = prev_op->fold_activation_backward();
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_pool_geom g = geom(batch_size);
    if (out_packed_) {
      unwrap(rh_pool2d_fwd_bf16_packed(&g, in_packed_->as_ptr(), out_packed_->as_mut_ptr(), out_halo_, context_->stream()),
             "pooling forward");
      return;
    }
    if (slot_) {
      unwrap(rh_pool2d_fwd_slot(&g, in_act_->as_ptr(), out_act_->as_mut_ptr(), slot_->as_mut_ptr(), context_->stream()),
             "pooling forward");
      return;
    }
    unwrap(rh_pool2d_fwd(&g, in_act_->as_ptr(), out_act_->as_mut_ptr(), argmax_ ? argmax_->as_mut_ptr() : nullptr,
                         context_->stream()), "pooling forward");
  }
  // A max-pool between two convolutions of a packed bf16 chain pools the packed activations.
  bool can_emit_packed() const override {
    return packed_chain_ && !out_packed_ && config_.pool_op == PoolOperation::Max && config_.in_dims.c % 8 == 0 &&
           prev_op_->can_emit_packed() &&
           rh_bf16_act_bytes((int)batch_cap_, (int)out_dims_.c, (int)out_dims_.h, (int)out_dims_.w, 0) > 0;
  }
  std::shared_ptr<DeviceBuffer<uint8_t>> emit_packed(int halo) override {
    const size_t bytes = rh_bf16_act_bytes((int)batch_cap_, (int)out_dims_.c, (int)out_dims_.h, (int)out_dims_.w, halo);
    if (!can_emit_packed() || !bytes) panic("Pool2dOperator: no packed output for this configuration");
    in_packed_ = prev_op_->emit_packed(0);
    out_packed_.reset(new DeviceBuffer<uint8_t>(bytes, context_));   // zero-filled: the border stays zero
    out_halo_ = halo;
    return out_packed_;
  }
  void backward(size_t batch_size) override {
    if (!in_delta_) return;
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_pool_geom g = geom(batch_size);
    if (slot_) {
      unwrap(rh_pool2d_bwd_slot(&g, fold_relu_ ? out_act_->as_ptr() : nullptr, out_delta_->as_ptr(), in_delta_->as_mut_ptr(),
                                slot_->as_ptr(), context_->stream()), "pooling backward");
      return;
    }
    if (fold_relu_ && config_.pool_op == PoolOperation::Average) {
      unwrap(rh_pool2d_bwd_avg_relu(&g, in_act_->as_ptr(), out_delta_->as_ptr(), in_delta_->as_mut_ptr(), context_->stream()),
             "pooling backward");
      return;
    }
    if (fold_relu_) {
      unwrap(rh_pool2d_bwd_relu(&g, out_act_->as_ptr(), out_delta_->as_ptr(), in_delta_->as_mut_ptr(), argmax_->as_ptr(),
                                context_->stream()), "pooling backward");
      return;
    }
    unwrap(rh_pool2d_bwd(&g, in_act_->as_ptr(), out_act_->as_ptr(), out_delta_->as_ptr(), in_delta_->as_mut_ptr(),
                         argmax_ ? argmax_->as_ptr() : nullptr, context_->stream()), "pooling backward");
  }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) {
      if (out_packed_)
        unwrap(rh_bf16_unpack_nchw((int)batch_cap_, (int)out_dims_.c, (int)out_dims_.h, (int)out_dims_.w, out_halo_,
                                   out_packed_->as_ptr(), out_act_->as_mut_ptr(), context_->stream()), "bf16 unpack");
      *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true;
    }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    return false;
  }
  const char* kind() const override { return "Pool2dOperator"; }

 private:
  rh_pool_geom geom(size_t batch) const {
    rh_pool_geom g;
    g.N = (int)batch; g.C = (int)config_.in_dims.c; g.H = (int)config_.in_dims.h; g.W = (int)config_.in_dims.w;
    g.size = (int)config_.pool_size; g.stride = (int)config_.pool_stride; g.pad = (int)config_.pool_pad;
    g.mode = config_.pool_op == PoolOperation::Max ? RH_POOL_MAX : RH_POOL_AVG_INCL_PAD;
    g.round = config_.ceil_mode ? RH_ROUND_CEIL : RH_ROUND_FLOOR;
    return g;
  }
  size_t batch_cap_;
  Pool2dOperatorConfig config_;
  Ctx context_;
  Dims3 out_dims_;
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  std::unique_ptr<DeviceBuffer<int32_t>> argmax_;   // private arg-max mask, one of the two forms
  std::unique_ptr<DeviceBuffer<uint8_t>> slot_;
  bool fold_relu_ = false;  // backward also applies the producer's ReLU mask
  Operator* prev_op_;       // (owned by the worker, which outlives this operator's use of it: construction only)
  bool packed_chain_;
  std::shared_ptr<DeviceBuffer<uint8_t>> in_packed_, out_packed_;
  int out_halo_ = 0;
};

// ---- DropoutOperator (src/operator/mod.rs:2134-2255) -------------------------------------------------------
// Training: rand_samples <- uniform [0,1) from the device generator, mask = rand > drop_ratio, out = in * mask
// (scale argument 1.0: no rescaling, as the reference passes it); Inference: a copy.
class DropoutOperator : public Operator {
 public:
  DropoutOperator(size_t batch_size, const DropoutOperatorConfig& config, const Operator* prev_op, Ctx context,
                  uint64_t seed, uint64_t stream_id)
      : batch_cap_(batch_size), config_(config), context_(context), seed_(seed), stream_id_(stream_id),
        rand_samples_(config.channels * batch_size, context), drop_mask_(config.channels * batch_size, context) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("DropoutOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.channels * batch_size);
    out_act_.reset(new DeviceBuffer<float>(config.channels * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(config.channels * batch_size, context));
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void forward(size_t batch_size, OpPhase phase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    rh_stream_t s = context_->stream();
    const size_t n = config_.channels * batch_size;
    if (!phase.training) {
      unwrap(rh_copy_d2d(out_act_->as_mut_ptr(), in_act_->as_ptr(), n * sizeof(float), s), "send");
      return;
    }
    last_first_ = next_first_;
    unwrap(rh_rng_fill_uniform01_device(seed_, stream_id_, next_first_, rand_samples_.as_mut_ptr(), n, s), "sample");
    next_first_ += n;
    rembrandt_kernel_map_dropout(in_act_->as_ptr(), (int32_t)n, config_.drop_ratio, 1.0f, rand_samples_.as_ptr(),
                                 out_act_->as_mut_ptr(), drop_mask_.as_mut_ptr(), s);
    unwrap_last("rembrandt_kernel_map_dropout");
  }
  void backward(size_t batch_size) override {
    if (!in_delta_) return;
    RB_ASSERT(batch_size <= batch_cap_);
    rembrandt_kernel_map_dropout_backprop(out_delta_->as_ptr(), (int32_t)(config_.channels * batch_size), config_.drop_ratio,
                                          1.0f, drop_mask_.as_ptr(), in_delta_->as_mut_ptr(), context_->stream());
    unwrap_last("rembrandt_kernel_map_dropout_backprop");
  }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    return false;
  }
  void stream(uint64_t* seed, uint64_t* stream_id, uint64_t* first) const {
    *seed = seed_; *stream_id = stream_id_; *first = last_first_;
  }
  const char* kind() const override { return "DropoutOperator"; }
  bool graph_safe(OpPhase phase) const override { return !phase.training; }  // a new piece of the uniform stream per step

 private:
  size_t batch_cap_;
  DropoutOperatorConfig config_;
  Ctx context_;
  uint64_t seed_, stream_id_, next_first_ = 0, last_first_ = 0;
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  DeviceBuffer<float> rand_samples_;
  DeviceBuffer<int32_t> drop_mask_;
};

// ---- LocalResNormOperator: cross-channel response normalisation (no counterpart operator in the reference) ----
class LocalResNormOperator : public Operator {
 public:
  LocalResNormOperator(size_t batch_size, const LocalResNormOperatorConfig& config, const Operator* prev_op, Ctx context)
      : batch_cap_(batch_size), config_(config), context_(context), denom_(config.in_dims.len() * batch_size, context) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("LocalResNormOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    RB_ASSERT(config.cross_size > 0 && config.min_div > 0.0f);
    out_act_.reset(new DeviceBuffer<float>(config.in_dims.len() * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(config.in_dims.len() * batch_size, context));
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_lrn_geom g = geom(batch_size);
    unwrap(rh_lrn_fwd(&g, in_act_->as_ptr(), out_act_->as_mut_ptr(), denom_.as_mut_ptr(), context_->stream()), "lrn forward");
  }
  void backward(size_t batch_size) override {
    if (!in_delta_) return;
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_lrn_geom g = geom(batch_size);
    unwrap(rh_lrn_bwd(&g, in_act_->as_ptr(), out_act_->as_ptr(), denom_.as_ptr(), out_delta_->as_ptr(),
                      in_delta_->as_mut_ptr(), context_->stream()), "lrn backward");
  }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    return false;
  }
  const char* kind() const override { return "LocalResNormOperator"; }

 private:
  rh_lrn_geom geom(size_t batch) const {
    rh_lrn_geom g;
    g.N = (int)batch; g.C = (int)config_.in_dims.c; g.H = (int)config_.in_dims.h; g.W = (int)config_.in_dims.w;
    g.size = (int)config_.cross_size; g.scale = config_.scale; g.power = config_.power; g.min_div = config_.min_div;
    return g;
  }
  size_t batch_cap_;
  LocalResNormOperatorConfig config_;
  Ctx context_;
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  DeviceBuffer<float> denom_;
};

// ---- conv (no bias) + spatial batch norm: the unit the three batch-normalised operators are made of ------------
// Buffers and update rules per unit as in src/operator/conv.rs:133-160 (buffers), :640-911 (regularize on the
// filter only; accumulate / update / save / restore / reset on filter, scale and bias; the moving statistics are
// saved and restored with the parameters).
struct BNormConvUnit {
  typedef std::unique_ptr<DeviceBuffer<float>> Buf;
  Dims3 in_dims, out_dims;
  size_t conv_size = 0, conv_stride = 1, conv_pad = 0, wlen = 0, chans = 0, batch_cap = 0;
  Ctx ctx;
  Buf weights, grad_weights, acc_grad_weights, save_weights;
  Buf scale, bias, scale_grad, bias_grad, acc_scale_grad, acc_bias_grad, save_scale, save_bias;
  Buf running_mean, running_ivar, save_running_mean, save_running_ivar, cached_mean, cached_ivar;
  Buf pre_act, pre_delta;  // the conv output the batch norm reads, and the gradient w.r.t. it
  bool backward = false;
  int conv_algo = 0;       // RH_ALGO_* bits of the unit's convolution calls
  bool beside = false;     // the last backward_params put the filter gradient on the second stream: the data gradient runs beside it

  void alloc(size_t batch, Dims3 in, size_t size, size_t stride, size_t pad, size_t out_channels, bool bwd, Ctx c) {
    in_dims = in; conv_size = size; conv_stride = stride; conv_pad = pad; chans = out_channels; ctx = c; backward = bwd;
    batch_cap = batch;
    out_dims = {out_dim_floor(in.w, size, stride, pad), out_dim_floor(in.h, size, stride, pad), out_channels};
    wlen = size * size * in.c * out_channels;
    auto mk = [&](size_t n) { return Buf(new DeviceBuffer<float>(n, c)); };
    weights = mk(wlen);
    scale = mk(chans); bias = mk(chans); running_mean = mk(chans); running_ivar = mk(chans);
    cached_mean = mk(chans); cached_ivar = mk(chans);
    scale_grad = mk(chans); bias_grad = mk(chans); acc_scale_grad = mk(chans); acc_bias_grad = mk(chans);
    save_scale = mk(chans); save_bias = mk(chans); save_running_mean = mk(chans); save_running_ivar = mk(chans);
    pre_act = mk(out_dims.len() * batch);
    if (bwd) {
      grad_weights = mk(wlen); acc_grad_weights = mk(wlen); save_weights = mk(wlen);
      pre_delta = mk(out_dims.len() * batch);
    }
  }
  rh_conv_geom geom(size_t batch) const {
    rh_conv_geom g;
    g.N = (int)batch; g.C = (int)in_dims.c; g.H = (int)in_dims.h; g.W = (int)in_dims.w;
    g.K = (int)chans; g.R = g.S = (int)conv_size; g.stride = (int)conv_stride; g.pad = (int)conv_pad;
    return g;
  }
  int plane() const { return (int)(out_dims.w * out_dims.h); }
  size_t workspace_bytes() const {
    const rh_conv_geom g = geom(batch_cap);
    size_t ws = std::max(conv_ws_upto(g, RH_CONV_FWD), bnorm_ws_upto(g.N, g.K, plane()));
    if (backward) {
      ws = std::max(ws, conv_ws_upto(g, RH_CONV_BWD_FILTER));
      ws = std::max(ws, conv_ws_upto(g, RH_CONV_BWD_DATA));
    }
    return ws;
  }
  rh_stream_t s() const { return ctx->stream(); }
  void fill(DeviceBuffer<float>& b, float v) { unwrap(rh_memset_f32(b.as_mut_ptr(), v, b.len(), s()), "set_constant"); }

  // Filter from the seeded generator (fan-in = size*size*in channels); scale 1, bias 0, moving mean 0, moving
  // inverse deviation 1 (src/operator/conv.rs:292-345).
  void init(const ParamsInit& init, uint64_t seed, uint64_t stream_id, const char* who) {
    std::vector<float> w(wlen);
    const size_t fan_in = conv_size * conv_size * in_dims.c;
    switch (init.kind) {
      case ParamsInit::Disabled: panic(std::string(who) + ": params init explicitly disabled");
      case ParamsInit::Uniform:
        unwrap(rh_rng_fill_uniform(seed, stream_id, w.data(), wlen, -init.value, init.value), "rh_rng_fill_uniform");
        break;
      case ParamsInit::Normal:
        unwrap(rh_rng_fill_normal(seed, stream_id, w.data(), wlen, 0.0f, init.value), "rh_rng_fill_normal");
        break;
      case ParamsInit::Xavier: panic(std::string(who) + ": Xavier init is unimplemented for this operator");
      case ParamsInit::KaimingFwd:
        unwrap(rh_rng_fill_normal(seed, stream_id, w.data(), wlen, 0.0f, (float)std::sqrt(2.0 / (double)fan_in)),
               "rh_rng_fill_normal");
        break;
    }
    weights->sync_load(w.data(), wlen);
    fill(*scale, 1.0f); fill(*bias, 0.0f); fill(*running_mean, 0.0f); fill(*running_ivar, 1.0f);
  }

  // out = beta_out*out + BN(conv(in)); `relu` clamps the blended result (the in-place rect that follows in the reference).
  void forward(size_t batch, const float* in, float* out, float beta_out, OpPhase phase, const BNormMovingAverage& avg,
               double epsilon, bool relu, DeviceBuffer<uint8_t>& ws, bool bf16) {
    const rh_conv_geom g = geom(batch);
    unwrap(rh_conv2d_fwd(&g, 1.0f, in, weights->as_ptr(), 0.0f, pre_act->as_mut_ptr(), nullptr, ws.as_mut_ptr(), ws.len(),
                         (bf16 ? RH_MATH_BF16_MFMA_FP32ACC : 0) | conv_algo, s()), "conv2d forward");
    const int flags = relu ? RH_FUSE_RELU : 0;
    if (phase.training) {
      if (!backward) panic("batch norm training missing backward operator");
      unwrap(rh_bnorm_fwd_train(g.N, g.K, plane(), 1.0f, pre_act->as_ptr(), beta_out, out, avg.at_iter(phase.t), epsilon,
                                scale->as_ptr(), bias->as_ptr(), running_mean->as_mut_ptr(), running_ivar->as_mut_ptr(),
                                cached_mean->as_mut_ptr(), cached_ivar->as_mut_ptr(), ws.as_mut_ptr(), ws.len(), flags, s()),
             "batch norm forward training");
    } else {
      unwrap(rh_bnorm_fwd_infer(g.N, g.K, plane(), 1.0f, pre_act->as_ptr(), beta_out, out, epsilon, scale->as_ptr(),
                                bias->as_ptr(), running_mean->as_ptr(), running_ivar->as_ptr(), ws.as_mut_ptr(), ws.len(),
                                flags, s()), "batch norm forward inference");
    }
  }
  // pre_delta = dBN(out_delta) with the scale / bias gradients accumulated, then grad_weights += dconv(in, pre_delta).
  // With `ws_aux` the filter gradient goes to the context's second stream (scratch of its own) and overlaps whatever
  // the main stream does next with pre_delta (the data gradient); the worker joins at the end of backward.
  // `relu_masked`: out_delta has not been through the backward of the ReLU that followed this unit's batch norm
  // (forward with beta_out 0); the batch-norm backward applies that mask itself, from pre_act.
  void backward_params(size_t batch, const float* in, const float* out_delta, double epsilon, DeviceBuffer<uint8_t>& ws,
                       DeviceBuffer<uint8_t>* ws_aux, bool relu_masked = false) {
    RB_ASSERT(backward);
    const rh_conv_geom g = geom(batch);
    if (relu_masked)
      unwrap(rh_bnorm_bwd_relu(g.N, g.K, plane(), 1.0f, 0.0f, pre_act->as_ptr(), out_delta, pre_delta->as_mut_ptr(), 1.0f, 1.0f,
                               epsilon, scale->as_ptr(), bias->as_ptr(), scale_grad->as_mut_ptr(), bias_grad->as_mut_ptr(),
                               cached_mean->as_ptr(), cached_ivar->as_ptr(), ws.as_mut_ptr(), ws.len(), s()),
             "batch norm backward with ReLU mask");
    else
      unwrap(rh_bnorm_bwd(g.N, g.K, plane(), 1.0f, 0.0f, pre_act->as_ptr(), out_delta, pre_delta->as_mut_ptr(), 1.0f, 1.0f,
                          epsilon, scale->as_ptr(), scale_grad->as_mut_ptr(), bias_grad->as_mut_ptr(), cached_mean->as_ptr(),
                          cached_ivar->as_ptr(), ws.as_mut_ptr(), ws.len(), s()), "batch norm backward");
    rh_stream_t sg = s();
    DeviceBuffer<uint8_t>* wg = &ws;
    beside = ws_aux != nullptr;
    if (ws_aux) {
      ctx->fork();
      sg = ctx->aux_stream();
      wg = ws_aux;
    }
    unwrap(rh_conv2d_bwd_filter(&g, 1.0f, in, pre_delta->as_ptr(), 1.0f, grad_weights->as_mut_ptr(), wg->as_mut_ptr(),
                                wg->len(), conv_algo, sg), "conv2d backward filter");
  }
  size_t aux_workspace_bytes() const {
    const rh_conv_geom g = geom(batch_cap);
    return conv_ws_upto(g, RH_CONV_BWD_FILTER);
  }
  // in_delta = beta*in_delta + dconv^T(weights, pre_delta)
  void backward_data(size_t batch, float* in_delta, float beta, DeviceBuffer<uint8_t>& ws) {
    const rh_conv_geom g = geom(batch);
    unwrap(rh_conv2d_bwd_data(&g, 1.0f, weights->as_ptr(), pre_delta->as_ptr(), beta, in_delta, ws.as_mut_ptr(), ws.len(),
                              conv_algo | (beside ? RH_ALGO_SHARED_GPU : 0), s()), "conv2d backward data");
  }

  void axpy(float a, const DeviceBuffer<float>& x, DeviceBuffer<float>& y) {
    unwrap(rh_saxpy((int64_t)x.len(), a, x.as_ptr(), y.as_mut_ptr(), s()), "sum");
  }
  void scal(float a, DeviceBuffer<float>& x) { unwrap(rh_sscal((int64_t)x.len(), a, x.as_mut_ptr(), s()), "scale"); }
  void copy(DeviceBuffer<float>& dst, const DeviceBuffer<float>& src) {
    unwrap(rh_copy_d2d(dst.as_mut_ptr(), src.as_ptr(), src.len() * 4, s()), "send");
  }
  void regularize(Regularization reg) {
    RB_ASSERT(backward);
    RB_ASSERT(reg.l2_reg_coef >= 0.0f);
    if (reg.l2_reg_coef > 0.0f) axpy(reg.l2_reg_coef, *weights, *grad_weights);
  }
  void accumulate_grads(float sc, float momentum) {
    RB_ASSERT(backward);
    scal(momentum, *acc_grad_weights); axpy(sc, *grad_weights, *acc_grad_weights);
    scal(momentum, *acc_scale_grad); axpy(sc, *scale_grad, *acc_scale_grad);
    scal(momentum, *acc_bias_grad); axpy(sc, *bias_grad, *acc_bias_grad);
  }
  void update_params(float sc) {
    RB_ASSERT(backward);
    axpy(sc, *acc_grad_weights, *weights); axpy(sc, *acc_scale_grad, *scale); axpy(sc, *acc_bias_grad, *bias);
  }
  void update_params2(float grad_scale, float update_scale) {
    RB_ASSERT(backward);
    if (grad_scale != 0.0f) { axpy(grad_scale, *grad_weights, *weights); axpy(grad_scale, *scale_grad, *scale); axpy(grad_scale, *bias_grad, *bias); }
    if (update_scale != 0.0f) { axpy(update_scale, *acc_grad_weights, *weights); axpy(update_scale, *acc_scale_grad, *scale); axpy(update_scale, *acc_bias_grad, *bias); }
  }
  void save_params() {
    RB_ASSERT(backward);
    copy(*save_weights, *weights); copy(*save_scale, *scale); copy(*save_bias, *bias);
    copy(*save_running_mean, *running_mean); copy(*save_running_ivar, *running_ivar);
  }
  void restore_params() {
    RB_ASSERT(backward);
    copy(*weights, *save_weights); copy(*scale, *save_scale); copy(*bias, *save_bias);
    copy(*running_mean, *save_running_mean); copy(*running_ivar, *save_running_ivar);
  }
  void reset() {
    if (!backward) return;
    scal(0.0f, *grad_weights); scal(0.0f, *scale_grad); scal(0.0f, *bias_grad);
  }
  void fused_sgd_step(float l2, float sc, float momentum, float apply, rh_stream_t st = nullptr) {
    RB_ASSERT(backward);
    if (!st) st = s();
    unwrap(rh_sgd_momentum_step((int64_t)wlen, weights->as_mut_ptr(), grad_weights->as_mut_ptr(), acc_grad_weights->as_mut_ptr(),
                                l2, sc, momentum, apply, 1, st), "rh_sgd_momentum_step");
    unwrap(rh_sgd_momentum_step((int64_t)chans, scale->as_mut_ptr(), scale_grad->as_mut_ptr(), acc_scale_grad->as_mut_ptr(),
                                0.0f, sc, momentum, apply, 1, st), "rh_sgd_momentum_step");
    unwrap(rh_sgd_momentum_step((int64_t)chans, bias->as_mut_ptr(), bias_grad->as_mut_ptr(), acc_bias_grad->as_mut_ptr(),
                                0.0f, sc, momentum, apply, 1, st), "rh_sgd_momentum_step");
  }
  void sgd_tensors(float l2, std::vector<rh_sgd_tensor>& out) {   // weight decay on the filter only
    RB_ASSERT(backward);
    out.push_back({weights->as_mut_ptr(), grad_weights->as_mut_ptr(), acc_grad_weights->as_mut_ptr(), (int64_t)wlen, l2});
    out.push_back({scale->as_mut_ptr(), scale_grad->as_mut_ptr(), acc_scale_grad->as_mut_ptr(), (int64_t)chans, 0.0f});
    out.push_back({bias->as_mut_ptr(), bias_grad->as_mut_ptr(), acc_bias_grad->as_mut_ptr(), (int64_t)chans, 0.0f});
  }
  // Blobs: filter as (size*size*in channels, out channels), then four (1, out channels) rows
  // (src/operator/conv.rs:361-406 params: scale, bias, moving mean, moving inverse deviation;
  //  :408-459 state: momentum of filter, scale, bias, then the cached batch mean and inverse deviation).
  void encode(std::vector<uint8_t>& blob, const DeviceBuffer<float>& w, const DeviceBuffer<float>* const rows[4]) const {
    ctx->sync();
    std::vector<float> h(wlen);
    w.sync_store(h.data(), wlen);
    const size_t wd[2] = {wlen / chans, chans}, rd[2] = {1, chans};
    ndarray_serialize(blob, h.data(), wd, 2);
    for (int i = 0; i < 4; ++i) {
      std::vector<float> r(chans);
      rows[i]->sync_store(r.data(), chans);
      ndarray_serialize(blob, r.data(), rd, 2);
    }
  }
  size_t decode(const uint8_t* blob, size_t len, DeviceBuffer<float>& w, DeviceBuffer<float>* const rows[4], const char* who) {
    std::vector<size_t> dims;
    std::vector<float> data;
    size_t off = ndarray_deserialize(blob, len, &dims, &data);
    if (dims.size() != 2 || dims[0] != wlen / chans || dims[1] != chans) panic(std::string(who) + ": weights blob has the wrong bound");
    w.sync_load(data.data(), wlen);
    for (int i = 0; i < 4; ++i) {
      off += ndarray_deserialize(blob + off, len - off, &dims, &data);
      if (dims.size() != 2 || dims[0] != 1 || dims[1] != chans) panic(std::string(who) + ": batch norm blob has the wrong bound");
      rows[i]->sync_load(data.data(), chans);
    }
    return off;
  }
  void encode_params(std::vector<uint8_t>& blob) const {
    const DeviceBuffer<float>* const rows[4] = {scale.get(), bias.get(), running_mean.get(), running_ivar.get()};
    encode(blob, *weights, rows);
  }
  size_t decode_params(const uint8_t* blob, size_t len, const char* who) {
    DeviceBuffer<float>* const rows[4] = {scale.get(), bias.get(), running_mean.get(), running_ivar.get()};
    return decode(blob, len, *weights, rows, who);
  }
  void encode_state(std::vector<uint8_t>& blob) const {
    RB_ASSERT(backward);
    const DeviceBuffer<float>* const rows[4] = {acc_scale_grad.get(), acc_bias_grad.get(), cached_mean.get(), cached_ivar.get()};
    encode(blob, *acc_grad_weights, rows);
  }
  size_t decode_state(const uint8_t* blob, size_t len, const char* who) {
    RB_ASSERT(backward);
    DeviceBuffer<float>* const rows[4] = {acc_scale_grad.get(), acc_bias_grad.get(), cached_mean.get(), cached_ivar.get()};
    return decode(blob, len, *acc_grad_weights, rows, who);
  }
  bool buffer(int id, float** ptr, size_t* len) {
    DeviceBuffer<float>* b = nullptr;
    switch (id) {
      case 2: b = weights.get(); break;
      case 4: b = grad_weights.get(); break;
      case 6: b = acc_grad_weights.get(); break;
      case 8: b = scale.get(); break;
      case 9: b = bias.get(); break;
      case 10: b = scale_grad.get(); break;
      case 11: b = bias_grad.get(); break;
      case 12: b = running_mean.get(); break;
      case 13: b = running_ivar.get(); break;
      case 14: b = cached_mean.get(); break;
      case 15: b = cached_ivar.get(); break;
      case 16: b = acc_scale_grad.get(); break;
      case 17: b = acc_bias_grad.get(); break;
      case 18: b = pre_act.get(); break;
      case 19: b = pre_delta.get(); break;
      default: return false;
    }
    if (!b) return false;
    *ptr = b->as_mut_ptr();
    *len = b->len();
    return true;
  }
};

// Common part of the three batch-normalised operators: the units' parameter plumbing.
class BNormUnitsOperator : public Operator {
 public:
  BNormUnitsOperator(size_t batch_size, size_t n_units, const Operator* prev_op, Ctx context, ExecOptions opts, const char* who)
      : batch_cap_(batch_size), units_(n_units), context_(context), opts_(opts) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic(std::string(who) + " missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    for (auto& u : units_) u.conv_algo = opts.winograd ? 0 : RH_ALGO_DIRECT;
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void regularize(Regularization reg) override { for (auto& u : units_) u.regularize(reg); }
  void accumulate_grads(float scale, float momentum) override { for (auto& u : units_) u.accumulate_grads(scale, momentum); }
  void update_params(float scale) override { for (auto& u : units_) u.update_params(scale); }
  void update_params2(float g, float v) override { for (auto& u : units_) u.update_params2(g, v); }
  void save_params() override { for (auto& u : units_) u.save_params(); }
  void restore_params() override { for (auto& u : units_) u.restore_params(); }
  void reset() override { for (auto& u : units_) u.reset(); }
  // The second-generation layer set has no batch-normalised layers (src/layer_new.rs): its update rule is not defined here.
  void backward_scaled(size_t batch_size, float scale) override {
    if (scale != 1.0f) panic(std::string(kind()) + ": backward(batch, scale) is unimplemented for scale != 1");
    backward(batch_size);
  }
  void descend(float, float, bool) override { panic(std::string(kind()) + ": descend is unimplemented"); }
  void reset_gradients(float) override { panic(std::string(kind()) + ": reset_gradients is unimplemented"); }
  // On the second stream, like the plain convolution layers' updates, except for the network's first layer.
  void fused_sgd_step(float l2, float scale, float mu, float apply) override {
    rh_stream_t st = updates_on_second_stream() ? context_->aux_stream() : nullptr;
    for (auto& u : units_) u.fused_sgd_step(l2, scale, mu, apply, st);
  }
  void sgd_tensors(float l2, std::vector<rh_sgd_tensor>& out) override { for (auto& u : units_) u.sgd_tensors(l2, out); }
  bool updates_on_second_stream() const override { return workspace_aux_ && overlap_on_ && in_delta_; }
  void encode_params(std::vector<uint8_t>& blob) override { for (auto& u : units_) u.encode_params(blob); }
  size_t decode_params(const uint8_t* blob, size_t len) override {
    size_t off = 0;
    for (auto& u : units_) off += u.decode_params(blob + off, len - off, kind());
    return off;
  }
  void encode_state(std::vector<uint8_t>& blob) override { for (auto& u : units_) u.encode_state(blob); }
  size_t decode_state(const uint8_t* blob, size_t len) override {
    size_t off = 0;
    for (auto& u : units_) off += u.decode_state(blob + off, len - off, kind());
    return off;
  }
  void init_params(const uint64_t seed[2]) override {
    for (size_t u = 0; u < units_.size(); ++u) units_[u].init(init_weights_, seed[0], seed[1] + 0x9E3779B97F4A7C15ull * u, kind());
  }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    if (which == 30 && mid_act_) { *ptr = mid_act_->as_mut_ptr(); *len = mid_act_->len(); return true; }
    if (which == 31 && mid_delta_) { *ptr = mid_delta_->as_mut_ptr(); *len = mid_delta_->len(); return true; }
    const int u = which / 100;
    if (u < 0 || (size_t)u >= units_.size()) return false;
    return units_[(size_t)u].buffer(which % 100, ptr, len);
  }

 protected:
  void alloc_common(Dims3 out_dims, bool bwd) {
    out_act_.reset(new DeviceBuffer<float>(out_dims.len() * batch_cap_, context_));
    out_delta_.reset(new DeviceBuffer<float>(out_dims.len() * batch_cap_, context_));
    size_t ws = 256;
    for (auto& u : units_) ws = std::max(ws, u.workspace_bytes());
    workspace_.reset(new DeviceBuffer<uint8_t>(ws, context_));
    if (bwd && opts_.overlap_backward) {
      size_t wa = 256;
      for (auto& u : units_) wa = std::max(wa, u.aux_workspace_bytes());
      workspace_aux_.reset(new DeviceBuffer<uint8_t>(wa, context_));
    }
  }
  // scratch of the filter gradients when they run on the second stream, else null
  DeviceBuffer<uint8_t>* aux_ws() { return workspace_aux_ && overlap_on_ ? workspace_aux_.get() : nullptr; }
  // ReLU after a batch norm: inside its apply kernel, or as the separate in-place pass of the reference.
  bool fuse_relu(ActivationFunction f) const {
    if (f != ActivationFunction::Identity && f != ActivationFunction::Rect) panic("unimplemented activation function");
    return f == ActivationFunction::Rect && opts_.fuse_epilogue;
  }
  void rect_after(ActivationFunction f, DeviceBuffer<float>& act, size_t frame_len, size_t batch) {
    if (!opts_.fuse_epilogue) apply_rect(f, act.as_mut_ptr(), frame_len, batch, context_->stream());
  }
  size_t batch_cap_;
  std::vector<BNormConvUnit> units_;
  Ctx context_;
  ExecOptions opts_;
  ParamsInit init_weights_ = ParamsInit::MakeDisabled();
  BNormMovingAverage mov_avg_ = BNormMovingAverage::MakeCumulative();
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  std::unique_ptr<DeviceBuffer<float>> mid_act_, mid_delta_;
  std::unique_ptr<DeviceBuffer<uint8_t>> workspace_, workspace_aux_;
  bool overlap_on_ = true;

 public:
  void set_overlap_backward(bool on) override { overlap_on_ = on; }
  // the weight of the newest batch in the moving statistics is a launch argument: constant only for the exponential
  // average after its first step
  bool graph_safe(OpPhase phase) const override {
    return !phase.training || (mov_avg_.kind == BNormMovingAverage::Exponential && phase.t > 0);
  }
};

// ---- BNormConv2dOperator (src/operator/conv.rs:106-912) ---------------------------------------------------
class BNormConv2dOperator : public BNormUnitsOperator {
 public:
  BNormConv2dOperator(size_t batch_size, OpCapability capability, const BNormConv2dOperatorConfig& config, const Operator* prev_op,
                      Ctx context, ExecOptions opts)
      : BNormUnitsOperator(batch_size, 1, prev_op, context, opts, "BNormConv2dOperator"), config_(config) {
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    init_weights_ = config.init_weights;
    mov_avg_ = config.bnorm_mov_avg;
    units_[0].alloc(batch_size, config.in_dims, config.conv_size, config.conv_stride, config.conv_pad, config.out_channels,
                    backward_enabled(capability), context);
    alloc_common(units_[0].out_dims, backward_enabled(capability));
  }
  void forward(size_t batch_size, OpPhase phase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    BNormConvUnit& u = units_[0];
    u.forward(batch_size, in_act_->as_ptr(), out_act_->as_mut_ptr(), 0.0f, phase, config_.bnorm_mov_avg, config_.bnorm_epsilon,
              fuse_relu(config_.act_func), *workspace_, opts_.bf16_forward);
    rect_after(config_.act_func, *out_act_, u.out_dims.len(), batch_size);
  }
  void backward(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    BNormConvUnit& u = units_[0];
    if (!act_bwd_folded_)
      apply_rect_backprop(config_.act_func, out_act_->as_ptr(), u.out_dims.len(), batch_size, out_delta_->as_mut_ptr(), context_->stream());
    u.backward_params(batch_size, in_act_->as_ptr(), out_delta_->as_ptr(), config_.bnorm_epsilon, *workspace_,
                      in_delta_ ? aux_ws() : nullptr);  // nothing to overlap with when no data gradient follows
    if (in_delta_) u.backward_data(batch_size, in_delta_->as_mut_ptr(), 0.0f, *workspace_);
  }
  const char* kind() const override { return "BNormConv2dOperator"; }
  bool fold_activation_backward() override {
    if (config_.act_func != ActivationFunction::Rect) return false;
    act_bwd_folded_ = true;
    return true;
  }

 private:
  bool act_bwd_folded_ = false;
  BNormConv2dOperatorConfig config_;
};

// ---- StackResConv2dOperator (src/operator/conv.rs:937-2182) -----------------------------------------------
// forward (:1497-1672): out <- in; mid = act(BN1(conv1(in))); out += BN2(conv2(mid)); out = act(out).
// backward (:1674-1830): mask out_delta; unit 2 gradients, mid_delta = conv2^T; mask mid_delta; unit 1 gradients;
// in_delta <- out_delta; in_delta += conv1^T.
class StackResConv2dOperator : public BNormUnitsOperator {
 public:
  StackResConv2dOperator(size_t batch_size, OpCapability capability, const StackResConv2dOperatorConfig& config,
                         const Operator* prev_op, Ctx context, ExecOptions opts)
      : BNormUnitsOperator(batch_size, 2, prev_op, context, opts, "StackResConv2dOperator"), config_(config) {
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    init_weights_ = config.init_weights;
    mov_avg_ = config.bnorm_mov_avg;
    const bool bwd = backward_enabled(capability);
    for (auto& u : units_) u.alloc(batch_size, config.in_dims, 3, 1, 1, config.in_dims.c, bwd, context);
    alloc_common(config.in_dims, bwd);
    mid_act_.reset(new DeviceBuffer<float>(config.in_dims.len() * batch_size, context));
    if (bwd) mid_delta_.reset(new DeviceBuffer<float>(config.in_dims.len() * batch_size, context));
  }
  void forward(size_t batch_size, OpPhase phase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const size_t len = config_.in_dims.len();
    const bool fuse = fuse_relu(config_.act_func);
    units_[0].forward(batch_size, in_act_->as_ptr(), mid_act_->as_mut_ptr(), 0.0f, phase, config_.bnorm_mov_avg,
                      config_.bnorm_epsilon, fuse, *workspace_, opts_.bf16_forward);
    rect_after(config_.act_func, *mid_act_, len, batch_size);
    unwrap(rh_copy_d2d(out_act_->as_mut_ptr(), in_act_->as_ptr(), len * batch_size * 4, context_->stream()), "send");
    units_[1].forward(batch_size, mid_act_->as_ptr(), out_act_->as_mut_ptr(), 1.0f, phase, config_.bnorm_mov_avg,
                      config_.bnorm_epsilon, fuse, *workspace_, opts_.bf16_forward);
    rect_after(config_.act_func, *out_act_, len, batch_size);
  }
  void backward(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    RB_ASSERT((bool)mid_delta_);
    const size_t len = config_.in_dims.len();
    rh_stream_t s = context_->stream();
    apply_rect_backprop(config_.act_func, out_act_->as_ptr(), len, batch_size, out_delta_->as_mut_ptr(), s);
    units_[1].backward_params(batch_size, mid_act_->as_ptr(), out_delta_->as_ptr(), config_.bnorm_epsilon, *workspace_, aux_ws());
    units_[1].backward_data(batch_size, mid_delta_->as_mut_ptr(), 0.0f, *workspace_);
    // with fused epilogues the ReLU mask of mid is applied inside unit 0's batch-norm backward (mid_delta keeps the
    // unmasked values); otherwise in place, as the reference does
    const bool fold_mid = opts_.fuse_epilogue && config_.act_func == ActivationFunction::Rect;
    if (!fold_mid) apply_rect_backprop(config_.act_func, mid_act_->as_ptr(), len, batch_size, mid_delta_->as_mut_ptr(), s);
    units_[0].backward_params(batch_size, in_act_->as_ptr(), mid_delta_->as_ptr(), config_.bnorm_epsilon, *workspace_, aux_ws(),
                              fold_mid);
    if (in_delta_) {
      unwrap(rh_copy_d2d(in_delta_->as_mut_ptr(), out_delta_->as_ptr(), len * batch_size * 4, s), "send");
      units_[0].backward_data(batch_size, in_delta_->as_mut_ptr(), 1.0f, *workspace_);
    }
  }
  const char* kind() const override { return "StackResConv2dOperator"; }

 private:
  StackResConv2dOperatorConfig config_;
};

// ---- ProjStackResConv2dOperator (src/operator/conv.rs:2210-3560) ------------------------------------------
// forward (:2935-3172): mid = act(BN1(conv1(in))); out = BN2(conv2(mid)); out += BN3(conv3(in)); out = act(out).
// backward (:3174-3385): mask out_delta; unit 2 gradients, mid_delta = conv2^T; mask mid_delta; unit 1 gradients;
// unit 3 gradients from out_delta; in_delta = conv1^T; in_delta += conv3^T.
class ProjStackResConv2dOperator : public BNormUnitsOperator {
 public:
  ProjStackResConv2dOperator(size_t batch_size, OpCapability capability, const ProjStackResConv2dOperatorConfig& config,
                             const Operator* prev_op, Ctx context, ExecOptions opts)
      : BNormUnitsOperator(batch_size, 3, prev_op, context, opts, "ProjStackResConv2dOperator"), config_(config) {
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    init_weights_ = config.init_weights;
    mov_avg_ = config.bnorm_mov_avg;
    const Dims3 in = config.in_dims, out = config.out_dims;
    size_t stride;
    if (in.w == out.w && in.h == out.h) stride = 1;
    else if (in.w == 2 * out.w && in.h == 2 * out.h) stride = 2;
    else panic("ProjStackResConv2dOperator: the output extent must equal or halve the input extent");
    const bool bwd = backward_enabled(capability);
    units_[0].alloc(batch_size, in, 3, stride, 1, out.c, bwd, context);
    units_[1].alloc(batch_size, out, 3, 1, 1, out.c, bwd, context);
    units_[2].alloc(batch_size, in, 1, stride, 0, out.c, bwd, context);
    for (auto& u : units_) RB_ASSERT(u.out_dims.w == out.w && u.out_dims.h == out.h);
    alloc_common(out, bwd);
    mid_act_.reset(new DeviceBuffer<float>(out.len() * batch_size, context));
    if (bwd) mid_delta_.reset(new DeviceBuffer<float>(out.len() * batch_size, context));
  }
  void forward(size_t batch_size, OpPhase phase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const size_t len = config_.out_dims.len();
    const bool fuse = fuse_relu(config_.act_func);
    units_[0].forward(batch_size, in_act_->as_ptr(), mid_act_->as_mut_ptr(), 0.0f, phase, config_.bnorm_mov_avg,
                      config_.bnorm_epsilon, fuse, *workspace_, opts_.bf16_forward);
    rect_after(config_.act_func, *mid_act_, len, batch_size);
    units_[1].forward(batch_size, mid_act_->as_ptr(), out_act_->as_mut_ptr(), 0.0f, phase, config_.bnorm_mov_avg,
                      config_.bnorm_epsilon, false, *workspace_, opts_.bf16_forward);
    units_[2].forward(batch_size, in_act_->as_ptr(), out_act_->as_mut_ptr(), 1.0f, phase, config_.bnorm_mov_avg,
                      config_.bnorm_epsilon, fuse, *workspace_, opts_.bf16_forward);
    rect_after(config_.act_func, *out_act_, len, batch_size);
  }
  void backward(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    RB_ASSERT((bool)mid_delta_);
    const size_t len = config_.out_dims.len();
    rh_stream_t s = context_->stream();
    apply_rect_backprop(config_.act_func, out_act_->as_ptr(), len, batch_size, out_delta_->as_mut_ptr(), s);
    units_[1].backward_params(batch_size, mid_act_->as_ptr(), out_delta_->as_ptr(), config_.bnorm_epsilon, *workspace_, aux_ws());
    units_[1].backward_data(batch_size, mid_delta_->as_mut_ptr(), 0.0f, *workspace_);
    // with fused epilogues the ReLU mask of mid is applied inside unit 0's batch-norm backward (mid_delta keeps the
    // unmasked values); otherwise in place, as the reference does
    const bool fold_mid = opts_.fuse_epilogue && config_.act_func == ActivationFunction::Rect;
    if (!fold_mid) apply_rect_backprop(config_.act_func, mid_act_->as_ptr(), len, batch_size, mid_delta_->as_mut_ptr(), s);
    units_[0].backward_params(batch_size, in_act_->as_ptr(), mid_delta_->as_ptr(), config_.bnorm_epsilon, *workspace_, aux_ws(),
                              fold_mid);
    units_[2].backward_params(batch_size, in_act_->as_ptr(), out_delta_->as_ptr(), config_.bnorm_epsilon, *workspace_, aux_ws());
    if (in_delta_) {
      units_[0].backward_data(batch_size, in_delta_->as_mut_ptr(), 0.0f, *workspace_);
      units_[2].backward_data(batch_size, in_delta_->as_mut_ptr(), 1.0f, *workspace_);
    }
  }
  const char* kind() const override { return "ProjStackResConv2dOperator"; }

 private:
  ProjStackResConv2dOperatorConfig config_;
};

// ---- SoftmaxKLLossOperator ------------------------------------------------------------------------------
class SoftmaxKLLossOperator : public LossOperator {
 public:
  SoftmaxKLLossOperator(size_t batch_size, const CategoricalLossConfig& loss_config, const Operator* prev_op, Ctx context)
      : batch_cap_(batch_size), loss_config_(loss_config), context_(context),
        label_cats_(batch_size, context), label_cats_h_(batch_size, 0), weights_(batch_size, context),
        weights_h_(batch_size, 0.0f), out_values_(loss_config.num_categories * batch_size, context),
        max_value_(batch_size, context), out_cats_(batch_size, context), out_cats_h_(batch_size, 0),
        out_loss1_(batch_size, context), out_loss_(1, context), acc_loss_(1, context), step_counter_(1, context),
        readback_((batch_size + 1) * 4, context) {
    RB_ASSERT(prev_op != nullptr);
    unwrap(rh_memset_f32(step_counter_.as_mut_ptr(), 0.0f, 1, context_->stream()), "set_constant");
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("SoftmaxKLLossOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_delta_ != nullptr);
    RB_ASSERT(in_act_->len() >= loss_config.num_categories * batch_size);
  }
  size_t batch_size() const override { return batch_cap_; }
  void forward(size_t batch_size, OpPhase phase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    step_valid_ = 0;
    if (armed_ && phase.training) {
      unwrap(rh_softmax_kl_step(in_act_->as_ptr(), (int)loss_config_.num_categories, (int)batch_size, label_cats_.as_ptr(),
                                weights_.as_ptr(), out_values_.as_mut_ptr(), max_value_.as_mut_ptr(), out_cats_.as_mut_ptr(),
                                out_loss1_.as_mut_ptr(), out_loss_.as_mut_ptr(),
                                in_delta_->as_mut_ptr(), reinterpret_cast<uint32_t*>(step_counter_.as_mut_ptr()),
                                context_->stream()), "softmax / loss step");
      step_valid_ = batch_size;
      return;
    }
    unwrap(rh_softmax_fwd(in_act_->as_ptr(), out_values_.as_mut_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                          context_->stream()), "softmax forward");
  }
  bool arm_train_step(bool on) override {
    armed_ = on;
    if (!on) step_valid_ = 0;
    return true;
  }
  void backward(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    if (step_valid_ == batch_size && batch_size > 0) return;   // forward() already left the delta in in_delta_
    rembrandt_kernel_batch_map_softmax_kl_backward(out_values_.as_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                                                   label_cats_.as_ptr(), weights_.as_ptr(), in_delta_->as_mut_ptr(),
                                                   context_->stream());
    unwrap_last("rembrandt_kernel_batch_map_softmax_kl_backward");
  }
  void stage_label(size_t batch_idx, int32_t category) override {
    RB_ASSERT(batch_idx < batch_cap_);
    RB_ASSERT(category >= 0 && (size_t)category < loss_config_.num_categories);  // src/opt/sgd/new.rs:296-299
    label_cats_h_[batch_idx] = category;
  }
  void load_labels(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    step_valid_ = 0;
    label_cats_.sync_load(label_cats_h_.data(), batch_cap_);
  }
  void stage_weight(size_t batch_idx, float weight) override {
    RB_ASSERT(batch_idx < batch_cap_);
    weights_h_[batch_idx] = weight;
  }
  void load_weights(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    step_valid_ = 0;
    weights_.sync_load(weights_h_.data(), batch_cap_);
  }
  float store_loss(size_t batch_size) override {
    enqueue_loss(batch_size);
    return fetch_loss();
  }
  void enqueue_loss(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    if (step_valid_ == batch_size && batch_size > 0) return;
    rh_stream_t s = context_->stream();
    rembrandt_kernel_batch_map_softmax_kl_loss1(out_values_.as_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                                                label_cats_.as_ptr(), weights_.as_ptr(), 0.0f, out_loss1_.as_mut_ptr(), s);
    unwrap_last("rembrandt_kernel_batch_map_softmax_kl_loss1");
    rembrandt_kernel_batch_blockreduce_sum(out_loss1_.as_ptr(), (int)batch_size, 1, out_loss_.as_mut_ptr(), 0.0f, s);
    unwrap_last("rembrandt_kernel_batch_blockreduce_sum");
  }
  float fetch_loss() override {
    float h = 0.0f;
    out_loss_.sync_store(&h, 1);
    return h;
  }
  // Second generation (src/layer_new.rs:2103-2134): out_loss sums the batches' losses until reset_loss.  The
  // reference's per-sample kernel there (`..._softmax_cross_entropy_loss`, trailing argument 1.0) lives outside its
  // tree, so what that 1.0 means is this build's reading: loss1[n] = -w_n log p[n, y_n] is overwritten per batch
  // (kGen2Loss1Accumulate = 0: the kl_loss1 kernel with factor 0), then the block sum is added to out_loss with factor
  // 1.  The other reading (loss1 itself accumulates over the batches, which reset_loss zeroing out_loss1 hints at)
  // is kGen2Loss1Accumulate = 1; it would count every earlier batch's sample losses again in each later block sum.
  static constexpr float kGen2Loss1Accumulate = 0.0f;
  void reset_loss(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    rh_stream_t s = context_->stream();
    unwrap(rh_memset_f32(out_loss1_.as_mut_ptr(), 0.0f, batch_cap_, s), "set_constant");
    unwrap(rh_memset_f32(acc_loss_.as_mut_ptr(), 0.0f, 1, s), "set_constant");
  }
  void accumulate_loss(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    rh_stream_t s = context_->stream();
    rembrandt_kernel_batch_map_softmax_kl_loss1(out_values_.as_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                                                label_cats_.as_ptr(), weights_.as_ptr(), kGen2Loss1Accumulate,
                                                out_loss1_.as_mut_ptr(), s);
    unwrap_last("rembrandt_kernel_batch_map_softmax_kl_loss1");
    rembrandt_kernel_batch_blockreduce_sum(out_loss1_.as_ptr(), (int)batch_size, 1, acc_loss_.as_mut_ptr(), 1.0f, s);
    unwrap_last("rembrandt_kernel_batch_blockreduce_sum");
  }
  float store_accumulated_loss() override {
    float h = 0.0f;
    acc_loss_.sync_store(&h, 1);
    return h;
  }
  void store_output_categories(size_t batch_size) override {
    enqueue_output_categories(batch_size);
    fetch_output_categories(batch_size);
  }
  void enqueue_output_categories(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    if (step_valid_ == batch_size && batch_size > 0) return;
    rembrandt_kernel_batch_blockreduce_argmax(out_values_.as_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                                              max_value_.as_mut_ptr(), out_cats_.as_mut_ptr(), context_->stream());
    unwrap_last("rembrandt_kernel_batch_blockreduce_argmax");
  }
  void fetch_output_categories(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    out_cats_.sync_store(out_cats_h_.data(), batch_cap_);
  }
  void begin_fetch(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    unwrap(rh_store_begin(context_->raw(), readback_.data(), out_cats_.as_ptr(), batch_cap_ * 4), "store (categories)");
    unwrap(rh_store_begin(context_->raw(), readback_.data() + batch_cap_ * 4, out_loss_.as_ptr(), 4), "store (loss)");
  }
  float finish_fetch(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    unwrap(rh_store_wait(context_->raw()), "store wait");
    std::memcpy(out_cats_h_.data(), readback_.data(), batch_cap_ * 4);
    float h;
    std::memcpy(&h, readback_.data() + batch_cap_ * 4, 4);
    return h;
  }
  const int32_t* get_output_categories(size_t) const override { return out_cats_h_.data(); }
  size_t accuracy_count(size_t batch_size) const override {
    RB_ASSERT(batch_size <= batch_cap_);
    size_t correct = 0;
    for (size_t i = 0; i < batch_size; ++i) correct += label_cats_h_[i] == out_cats_h_[i];
    return correct;
  }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which != 0) return false;  // the softmax probabilities
    *ptr = out_values_.as_mut_ptr();
    *len = out_values_.len();
    return true;
  }
  const char* kind() const override { return "SoftmaxKLLossOperator"; }

 private:
  friend struct ::rembrandt::ClassifierTail;
  size_t batch_cap_;
  CategoricalLossConfig loss_config_;
  Ctx context_;
  SharedDeviceBuf in_act_, in_delta_;
  DeviceBuffer<int32_t> label_cats_;
  std::vector<int32_t> label_cats_h_;
  DeviceBuffer<float> weights_;
  std::vector<float> weights_h_;
  DeviceBuffer<float> out_values_, max_value_;
  DeviceBuffer<int32_t> out_cats_;
  bool armed_ = false;       // arm_train_step
  size_t step_valid_ = 0;    // batch size whose categories, loss and delta the last forward() produced; 0: none
  std::vector<int32_t> out_cats_h_;
  DeviceBuffer<float> out_loss1_, out_loss_, acc_loss_;
  DeviceBuffer<float> step_counter_;   // the one word rh_softmax_kl_step counts its blocks in (zero between calls)
  PinnedBytes readback_;  // categories, then the loss: what begin_fetch copies
};

}  // namespace

// ---- the classifier tail of a train step as two launches ---------------------------------------------------
// AffineOperator (ReLU or identity) -> AffineOperator (identity) -> SoftmaxKLLossOperator, of a size where one block
// holds a sample's whole chain (rh_affine2_softmax_kl_step_supported).  forward_train stands for the three
// operators' forward(), the loss operator's enqueue_* and backward(), and the data-gradient halves of the two
// affine backward() calls; backward_train for their parameter-gradient halves.  Every buffer the operators expose
// holds what the separate calls leave there (the first layer's delta after its activation's backward).
// A first layer too large for that (LeNet's 2450 x 500) keeps its three tiled products: from_h, where the fused
// kernels start from its output and stand for the second layer and the loss only.
struct ClassifierTail {
  AffineOperator* fc1;
  AffineOperator* fc2;
  SoftmaxKLLossOperator* loss;
  Ctx context;
  bool from_h = false;
  size_t replaced() const { return from_h ? 1 : 2; }   // hidden operators, counted from the end, whose calls it stands for

  static std::shared_ptr<ClassifierTail> detect(std::vector<std::unique_ptr<Operator>>& hidden, LossOperator* loss_op,
                                                size_t batch_cap, const ExecOptions& opts, Ctx context) {
    if (!opts.fuse_tail || !opts.fuse_epilogue || hidden.size() < 2) return nullptr;
    auto* a1 = dynamic_cast<AffineOperator*>(hidden[hidden.size() - 2].get());
    auto* a2 = dynamic_cast<AffineOperator*>(hidden[hidden.size() - 1].get());
    auto* l = dynamic_cast<SoftmaxKLLossOperator*>(loss_op);
    if (!a1 || !a2 || !l || !a1->params_.has_backward() || !a2->params_.has_backward()) return nullptr;
    if (a2->config_.act_func != ActivationFunction::Identity) return nullptr;
    if (a1->config_.act_func != ActivationFunction::Identity && a1->config_.act_func != ActivationFunction::Rect) return nullptr;
    if (a1->config_.out_channels != a2->config_.in_channels || a2->config_.out_channels != l->loss_config_.num_categories)
      return nullptr;
    const int H = (int)a1->config_.out_channels, C = (int)a2->config_.out_channels;
    const bool whole = rh_affine2_softmax_kl_step_supported((int)batch_cap, (int)a1->config_.in_channels, H, C) != 0;
    if (!whole && !rh_affine2_softmax_kl_step_supported((int)batch_cap, 0, H, C)) return nullptr;
    std::shared_ptr<ClassifierTail> t(new ClassifierTail());
    t->fc1 = a1; t->fc2 = a2; t->loss = l; t->context = context; t->from_h = !whole;
    return t;
  }
  bool updates_on_second_stream() const {
    return (!from_h && fc1->updates_on_second_stream()) || fc2->updates_on_second_stream();
  }
  void forward_train(size_t batch_size) {
    RB_ASSERT(batch_size <= fc1->batch_cap_);
    const int I = from_h ? 0 : (int)fc1->config_.in_channels, H = (int)fc1->config_.out_channels, C = (int)fc2->config_.out_channels;
    unwrap(rh_affine2_softmax_kl_step(
               (int)batch_size, I, H, C, fc1->config_.act_func == ActivationFunction::Rect ? 1 : 0,
               from_h ? nullptr : fc1->in_act_->as_ptr(),
               fc1->params_.weights->as_ptr(), fc1->params_.bias->as_ptr(), fc2->params_.weights->as_ptr(),
               fc2->params_.bias->as_ptr(), loss->label_cats_.as_ptr(), loss->weights_.as_ptr(), fc1->out_act_->as_mut_ptr(),
               fc2->out_act_->as_mut_ptr(), loss->out_values_.as_mut_ptr(), loss->max_value_.as_mut_ptr(),
               loss->out_cats_.as_mut_ptr(), loss->out_loss1_.as_mut_ptr(), loss->out_loss_.as_mut_ptr(),
               fc2->out_delta_->as_mut_ptr(), fc1->out_delta_->as_mut_ptr(),
               !from_h && fc1->in_delta_ ? fc1->in_delta_->as_mut_ptr() : nullptr,
               reinterpret_cast<uint32_t*>(loss->step_counter_.as_mut_ptr()), context->stream()),
           "classifier tail (forward, loss, data gradients)");
    loss->step_valid_ = batch_size;   // categories, loss and delta are there: the loss operator's calls launch nothing
  }
  void backward_train(size_t batch_size) {
    const int I = from_h ? 0 : (int)fc1->config_.in_channels, H = (int)fc1->config_.out_channels, C = (int)fc2->config_.out_channels;
    rh_stream_t sg = context->stream();
    if (from_h ? fc2->overlap_on_ : fc1->overlap_on_ && fc1->in_delta_) {   // as AffineOperator::backward places its parameter gradients
      context->fork();
      sg = context->aux_stream();
    }
    const float beta2 = fc2->params_.take_backward_beta();
    // (from h: the first layer's backward() follows and takes its beta itself; its bias gradient, the column sums of the
    // delta this launch reads anyway, is formed here with the same beta)
    const float beta1 = from_h ? (fc1->params_.grads_stale ? 0.0f : 1.0f) : fc1->params_.take_backward_beta();
    if (from_h) fc1->delta_masked_once_ = fc1->bias_grad_done_ = true;   // the delta it finds is the masked one
    unwrap(rh_affine2_bwd_params((int)batch_size, I, H, C, from_h ? nullptr : fc1->in_act_->as_ptr(), fc1->out_act_->as_ptr(),
                                 fc1->out_delta_->as_ptr(), fc2->out_delta_->as_ptr(), beta1,
                                 fc1->params_.grad_weights->as_mut_ptr(), fc1->params_.grad_bias->as_mut_ptr(), beta2,
                                 fc2->params_.grad_weights->as_mut_ptr(), fc2->params_.grad_bias->as_mut_ptr(), sg),
           "classifier tail (parameter gradients)");
  }
};

// ---- SequentialOperatorWorker ---------------------------------------------------------------------------
SequentialOperatorWorker::SequentialOperatorWorker(const SequentialOperatorConfig& config, size_t batch_size,
                                                   OpCapability capability, const uint64_t shared_seed[2],
                                                   std::shared_ptr<DeviceContext> context, ExecOptions opts)
    : batch_size_(batch_size), context_(context) {
  shared_seed_[0] = shared_seed[0];
  shared_seed_[1] = shared_seed[1];
  RB_ASSERT(batch_size > 0);
  if (!config.has_input || config.input_op.kind != OperatorConfig::Data3d) panic("SequentialOperatorWorker: missing input operator");
  if (!config.has_loss) panic("SequentialOperatorWorker: missing loss operator");
  const uint64_t input_seed[2] = {shared_seed[0] ^ 0x44617461336421ull, shared_seed[1] + 0x9E3779B97F4A7C15ull};
  input_op_.reset(new Data3dOperator(batch_size, config.input_op.data3d, context, input_seed));
  opts.bf16_packed_chain = opts.bf16_forward && !backward_enabled(capability);
  Operator* prev = input_op_.get();
  size_t params_off = 0;
  for (const auto& c : config.hidden_ops) {
    std::unique_ptr<Operator> op;
    switch (c.kind) {
      case OperatorConfig::Affine: op.reset(new AffineOperator(batch_size, capability, c.affine, prev, context, opts)); break;
      case OperatorConfig::Conv2d: op.reset(new Conv2dOperator(batch_size, capability, c.conv2d, prev, context, opts)); break;
      case OperatorConfig::Pool2d: op.reset(new Pool2dOperator(batch_size, c.pool2d, prev, context, opts)); break;
      case OperatorConfig::Dropout:
        op.reset(new DropoutOperator(batch_size, c.dropout, prev, context, shared_seed[0] ^ (shared_seed[1] << 32 | shared_seed[1] >> 32),
                                     0xD0000000ull + hidden_ops_.size()));
        break;
      case OperatorConfig::LocalResNorm: op.reset(new LocalResNormOperator(batch_size, c.lrn, prev, context)); break;
      case OperatorConfig::BNormConv2d:
        op.reset(new BNormConv2dOperator(batch_size, capability, c.bnorm_conv2d, prev, context, opts));
        break;
      case OperatorConfig::StackResConv2d:
        op.reset(new StackResConv2dOperator(batch_size, capability, c.stack_res_conv2d, prev, context, opts));
        break;
      case OperatorConfig::ProjStackResConv2d:
        op.reset(new ProjStackResConv2dOperator(batch_size, capability, c.proj_stack_res_conv2d, prev, context, opts));
        break;
      default: panic("SequentialOperatorWorker: not a hidden operator");
    }
    params_off += c.params_len();
    hidden_ops_.push_back(std::move(op));
    prev = hidden_ops_.back().get();
  }
  RB_ASSERT(params_off == config.params_len());  // src/operator/worker.rs:289
  loss_op_.reset(new SoftmaxKLLossOperator(batch_size, config.loss_op.loss, prev, context));
  if (backward_enabled(capability)) tail_ = ClassifierTail::detect(hidden_ops_, loss_op_.get(), batch_size, opts, context);
  context_->sync();
}

bool SequentialOperatorWorker::arm_train_step(bool on) {
  const bool armed = loss_op_->arm_train_step(on);
  tail_armed_ = on && armed && tail_ != nullptr;
  if (!on) tail_done_ = 0;
  return armed;
}

LossOperator* SequentialOperatorWorker::loss_operator(size_t rank) {
  RB_ASSERT(rank == 0);
  return loss_op_.get();
}

void SequentialOperatorWorker::settle() {
  if (aux_pending_) {
    context_->join();
    aux_pending_ = false;
  }
}

void SequentialOperatorWorker::init_params(const uint64_t shared_seed[2]) {
  settle();
  Xorshiftplus128 rng(shared_seed);
  for (auto& op : hidden_ops_) {
    const uint64_t op_seed[2] = {rng.next_u64(), rng.next_u64()};
    op->init_params(op_seed);
  }
}
void SequentialOperatorWorker::forward(size_t batch_size, OpPhase phase) {
  input_op_->forward(batch_size, phase);
  const bool tail = tail_armed_ && phase.training && batch_size > 0;
  const size_t n = hidden_ops_.size() - (tail ? tail_->replaced() : 0);
  for (size_t i = 0; i < n; ++i) {
    Operator* op = hidden_ops_[i].get();
    if (aux_pending_ && op->updates_on_second_stream()) settle();  // its parameters were updated on the second stream
    op->forward(batch_size, phase);
  }
  tail_done_ = 0;
  if (tail) {
    if (aux_pending_ && tail_->updates_on_second_stream()) settle();
    tail_->forward_train(batch_size);
    tail_done_ = batch_size;
    return;
  }
  loss_op_->forward(batch_size, phase);
}
void SequentialOperatorWorker::backward(size_t batch_size) {
  settle();
  size_t n = hidden_ops_.size();
  if (tail_armed_ && tail_done_ == batch_size && batch_size > 0) {
    tail_->backward_train(batch_size);   // the deltas are there since forward(): only the parameter gradients are left
    n -= tail_->replaced();
  } else {
    loss_op_->backward(batch_size);
  }
  tail_done_ = 0;
  for (size_t i = n; i-- > 0;) hidden_ops_[i]->backward(batch_size);
  context_->join();  // gradients computed on the second stream are complete for whatever the main stream does next
}
void SequentialOperatorWorker::regularize(Regularization reg) { settle(); for (auto& op : hidden_ops_) op->regularize(reg); }
void SequentialOperatorWorker::accumulate_grads(float scale, float momentum) { settle(); for (auto& op : hidden_ops_) op->accumulate_grads(scale, momentum); }
void SequentialOperatorWorker::update_params(float scale) { settle(); for (auto& op : hidden_ops_) op->update_params(scale); }
void SequentialOperatorWorker::update_params2(float g, float u) { settle(); for (auto& op : hidden_ops_) op->update_params2(g, u); }
void SequentialOperatorWorker::save_params() { settle(); for (auto& op : hidden_ops_) op->save_params(); }
void SequentialOperatorWorker::restore_params() { settle(); for (auto& op : hidden_ops_) op->restore_params(); }
void SequentialOperatorWorker::reset() { settle(); for (auto& op : hidden_ops_) op->reset(); }
void SequentialOperatorWorker::backward_scaled(size_t batch_size, float scale) {
  settle();
  loss_op_->backward(batch_size);  // the loss layer ignores the scale (src/layer_new.rs:1933)
  for (auto it = hidden_ops_.rbegin(); it != hidden_ops_.rend(); ++it) (*it)->backward_scaled(batch_size, scale);
  context_->join();
}
void SequentialOperatorWorker::descend(float scale, float l2_reg_coef, bool fused) {
  settle();
  for (auto& op : hidden_ops_) op->descend(scale, l2_reg_coef, fused);
}
void SequentialOperatorWorker::reset_gradients(float momentum) {
  settle();
  for (auto& op : hidden_ops_) op->reset_gradients(momentum);
}
bool SequentialOperatorWorker::graph_safe(OpPhase phase) const {
  if (!input_op_->graph_safe(phase) || !loss_op_->graph_safe(phase)) return false;
  for (const auto& op : hidden_ops_)
    if (!op->graph_safe(phase)) return false;
  return true;
}
void SequentialOperatorWorker::set_overlap_backward(bool on) {
  settle();
  context_->join();
  for (auto& op : hidden_ops_) op->set_overlap_backward(on);
}
std::vector<char> SequentialOperatorWorker::grad_state() const {
  std::vector<char> state(hidden_ops_.size());
  for (size_t i = 0; i < hidden_ops_.size(); ++i) state[i] = hidden_ops_[i]->grads_stale() ? 1 : 0;
  return state;
}
void SequentialOperatorWorker::set_grad_state(const std::vector<char>& state) {
  RB_ASSERT(state.size() == hidden_ops_.size());
  for (size_t i = 0; i < hidden_ops_.size(); ++i) hidden_ops_[i]->set_grads_stale(state[i] != 0);
}
void SequentialOperatorWorker::fused_sgd_step(float l2, float scale, float mu, float apply) {
  settle();
  // Operators that say so take their step on the second stream (forked here: it sees the finished gradients); the
  // next forward pass joins in front of the first of them, so these updates hide behind the layers before it.
  // All parameter blocks of a stream go in one launch: most of them are far too small to fill a launch of their own.
  std::vector<rh_sgd_tensor> on_main, on_aux;
  for (auto& op : hidden_ops_) op->sgd_tensors(l2, op->updates_on_second_stream() ? on_aux : on_main);
  RB_ASSERT(l2 >= 0.0f);
  if (!on_aux.empty()) {
    if (!aux_pending_) {
      context_->fork();
      aux_pending_ = true;
    }
    unwrap(rh_sgd_momentum_step_multi((int32_t)on_aux.size(), on_aux.data(), scale, mu, apply, 1, context_->aux_stream()),
           "rh_sgd_momentum_step_multi");
  }
  if (!on_main.empty())
    unwrap(rh_sgd_momentum_step_multi((int32_t)on_main.size(), on_main.data(), scale, mu, apply, 1, context_->stream()),
           "rh_sgd_momentum_step_multi");
}

void SequentialOperatorWorker::encode_params(std::vector<uint8_t>& blob) { settle(); for (auto& op : hidden_ops_) op->encode_params(blob); }
size_t SequentialOperatorWorker::decode_params(const uint8_t* blob, size_t len) {
  settle();
  size_t off = 0;
  for (auto& op : hidden_ops_) off += op->decode_params(blob + off, len - off);
  return off;
}
void SequentialOperatorWorker::encode_state(std::vector<uint8_t>& blob) {
  settle();
  for (auto& op : hidden_ops_) {  // params then momentum, operator by operator (gossip_dist.rs:1287-1291)
    op->encode_params(blob);
    op->encode_state(blob);
  }
}
size_t SequentialOperatorWorker::decode_state(const uint8_t* blob, size_t len) {
  settle();
  size_t off = 0;
  for (auto& op : hidden_ops_) {
    off += op->decode_params(blob + off, len - off);
    off += op->decode_state(blob + off, len - off);
  }
  return off;
}

namespace {
void make_dirs(const std::string& path) {  // create_dir_all; errors ignored as in the reference
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if (i == path.size() || path[i] == '/') {
      if (!cur.empty()) ::mkdir(cur.c_str(), 0777);
    }
    if (i < path.size()) cur.push_back(path[i]);
  }
}
void write_file(const std::string& path, const std::vector<uint8_t>& blob, const char* who) {
  std::ofstream f(path, std::ios::binary | std::ios::trunc);
  if (!f) panic(std::string(who) + ": failed to open blob file: " + path);
  f.write(reinterpret_cast<const char*>(blob.data()), (std::streamsize)blob.size());
  if (!f) panic(std::string(who) + ": failed to write to blob file: " + path);
}
std::vector<uint8_t> read_file(const std::string& path, const char* who) {
  std::ifstream f(path, std::ios::binary);
  if (!f) panic(std::string(who) + ": failed to open blob file: " + path);
  return std::vector<uint8_t>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}
}  // namespace

void SequentialOperatorWorker::checkpoint_params(size_t t, const std::string& prefix) {
  make_dirs(prefix);
  std::vector<uint8_t> blob;
  encode_params(blob);
  const std::string name = "params.t_" + std::to_string(t) + ".blob";
  write_file(prefix + "/" + name, blob, "checkpoint_params");
  const std::string latest = prefix + "/params.latest.blob";
  ::unlink(latest.c_str());
  if (::symlink(name.c_str(), latest.c_str()) != 0) panic("checkpoint_params: failed to symlink latest blob");
  const std::string ck = prefix + "/checkpoint";
  {
    std::ifstream old(ck, std::ios::binary);
    if (old) {
      std::ofstream bak(prefix + "/checkpoint.0", std::ios::binary | std::ios::trunc);
      bak << old.rdbuf();
    }
  }
  std::ofstream f(ck, std::ios::trunc);
  if (!f) panic("checkpoint_params: failed to open checkpoint file");
  f << t << "\n";
}

void SequentialOperatorWorker::checkpoint_state(const std::string& prefix) {
  make_dirs(prefix);
  std::vector<uint8_t> blob;
  encode_state(blob);
  write_file(prefix + "/state.latest.blob." + std::to_string(worker_rank()), blob, "checkpoint_state");
}

bool SequentialOperatorWorker::can_rollback(const std::string& prefix, size_t* t) const {
  std::ifstream f(prefix + "/checkpoint");
  if (!f) return false;
  std::string line;
  if (!std::getline(f, line)) return false;
  char* end = nullptr;
  const unsigned long long v = std::strtoull(line.c_str(), &end, 10);
  if (end == line.c_str()) return false;
  if (t) *t = (size_t)v;
  return true;
}

void SequentialOperatorWorker::rollback_params(const size_t* t, const std::string& prefix) {
  std::string path;
  if (t) {
    size_t latest = 0;
    if (!can_rollback(prefix, &latest)) panic("rollback_params: checkpoint file is missing or empty, but requested iter " + std::to_string(*t));
    RB_ASSERT(*t <= latest);
    path = prefix + "/params.t_" + std::to_string(*t) + ".blob";
  } else {
    path = prefix + "/params.latest.blob";
  }
  const std::vector<uint8_t> blob = read_file(path, "rollback_params");
  decode_params(blob.data(), blob.size());
}

void SequentialOperatorWorker::rollback_state(const std::string& prefix) {
  const std::vector<uint8_t> blob = read_file(prefix + "/state.latest.blob." + std::to_string(worker_rank()), "rollback_state");
  decode_state(blob.data(), blob.size());
}

bool SequentialOperatorWorker::dropout_stream(size_t hidden_idx, uint64_t* seed, uint64_t* stream_id, uint64_t* first) const {
  const DropoutOperator* d = dynamic_cast<const DropoutOperator*>(hidden_ops_.at(hidden_idx).get());
  if (!d) return false;
  d->stream(seed, stream_id, first);
  return true;
}

// ---- SGD policy -----------------------------------------------------------------------------------------
StepSizeSchedule StepSizeSchedule::MakeConstant(float s) {
  StepSizeSchedule sch = StepSizeSchedule();
  sch.kind = Constant;
  sch.step[0] = s;
  return sch;
}

float StepSizeSchedule::at_iter(size_t t) const {
  switch (kind) {
    case Constant: return step[0];
    case Anneal1: return t < iters[1] ? step[0] : step[1];
    case Anneal2: return t < iters[1] ? step[0] : t < iters[2] ? step[1] : step[2];
    case Anneal4:
      return t < iters[1] ? step[0] : t < iters[2] ? step[1] : t < iters[3] ? step[2] : t < iters[4] ? step[3] : step[4];
    case Decay: panic("StepSizeSchedule::Decay is unimplemented");  // as in the reference
    case Inverse: return step[0] / (1.0f + step[0] * step[1] * (float)t);
  }
  panic("bad StepSizeSchedule");
}

void SgdOpt::begin(Operator* op) {
  if (config_.momentum.kind == Momentum::UpdateNesterov) op->update_params(config_.momentum.mu);
  op->reset();
}

void SgdOpt::step(Operator* op, bool fused, bool defer_reapply) {
  const float l2 = config_.l2_reg_coef;
  const float step_size = config_.step_size.at_iter(iter_counter_);  // before the increment (StepSizeReference::Local)
  const float mu = config_.momentum.mu;
  const Momentum::Kind k = config_.momentum.kind;
  if (fused && (k == Momentum::Zero || k == Momentum::Update || k == Momentum::Gradient)) {
    iter_counter_ += 1;
    if (k == Momentum::Zero) op->fused_sgd_step(l2, -step_size, 0.0f, 1.0f);
    else if (k == Momentum::Update) op->fused_sgd_step(l2, -step_size, mu, 1.0f);
    else op->fused_sgd_step(l2, 1.0f, mu, -step_size);
    return;
  }
  op->regularize(Regularization::L2(l2));
  if (k == Momentum::UpdateNesterov && iter_counter_ > 0) op->update_params(-mu);
  iter_counter_ += 1;
  switch (k) {
    case Momentum::Zero: op->accumulate_grads(-step_size, 0.0f); break;
    case Momentum::Update:
    case Momentum::UpdateNesterov: op->accumulate_grads(-step_size, mu); break;
    case Momentum::Gradient:
    case Momentum::GradientNesterov: op->accumulate_grads(1.0f, mu); break;
  }
  switch (k) {
    case Momentum::Zero:
    case Momentum::Update:
    case Momentum::UpdateNesterov: op->update_params(1.0f); break;
    case Momentum::Gradient: op->update_params(-step_size); break;
    case Momentum::GradientNesterov: op->update_params2(-step_size, -step_size * mu); break;
  }
  op->reset();
  if (k == Momentum::UpdateNesterov && !defer_reapply) op->update_params(mu);
}

void SgdOptimization::begin(SequentialOperatorWorker* w) {
  w->reset_gradients(0.0f);
  w->loss_operator(0)->reset_loss(w->batch_size());
  t_ = 0;
}
void SgdOptimization::batch(SequentialOperatorWorker* w, size_t batch_size) {
  w->forward(batch_size, OpPhase::Training(t_));
  w->backward_scaled(batch_size, 1.0f);
  w->loss_operator(0)->accumulate_loss(batch_size);
}
void SgdOptimization::end_minibatch(SequentialOperatorWorker* w, bool fused) {
  const float descent_scale = config_.step_size.at_iter(t_) / (float)config_.minibatch_size;
  w->descend(descent_scale, config_.l2_reg_coef, fused);
  w->reset_gradients(config_.momentum);
  t_ += 1;
}

void SgdOpt::reapply(Operator* op) {
  if (config_.momentum.kind == Momentum::UpdateNesterov) op->update_params(config_.momentum.mu);
}

}  // namespace rembrandt
