// Host-side operator layer (see operator.hpp).  Uses only the C ABI of rembrandt_hip.h.
#include "operator.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>

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

Dims3 Pool2dOperatorConfig::get_out_dims() const {
  const int r = ceil_mode ? RH_ROUND_CEIL : RH_ROUND_FLOOR;
  return {(size_t)rh_pool2d_out_dim((int)in_dims.w, (int)pool_size, (int)pool_stride, (int)pool_pad, r),
          (size_t)rh_pool2d_out_dim((int)in_dims.h, (int)pool_size, (int)pool_stride, (int)pool_pad, r), in_dims.c};
}

size_t OperatorConfig::params_len() const {
  switch (kind) {
    case Affine: return affine.params_len();
    case Conv2d: return conv2d.params_len();
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

struct ParamTensors {
  std::unique_ptr<DeviceBuffer<float>> weights, bias;
  // backward-capable operators only
  std::unique_ptr<DeviceBuffer<float>> grad_weights, grad_bias, acc_grad_weights, acc_grad_bias, save_weights, save_bias;
  size_t wlen = 0, blen = 0;
  Ctx ctx;

  void alloc(size_t wl, size_t bl, bool backward, Ctx c) {
    wlen = wl; blen = bl; ctx = c;
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
    if (reg.l2_reg_coef > 0.0f) {
      unwrap(rh_saxpy((int64_t)wlen, reg.l2_reg_coef, weights->as_ptr(), grad_weights->as_mut_ptr(), s()), "matrix_sum");
      unwrap(rh_saxpy((int64_t)blen, reg.l2_reg_coef, bias->as_ptr(), grad_bias->as_mut_ptr(), s()), "row_vector_sum");
    }
  }
  // v = momentum*v; v += scale*g (src/operator/mod.rs:1195-1207)
  void accumulate_grads(float scale, float momentum) {
    RB_ASSERT(has_backward());
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
    unwrap(rh_sscal((int64_t)wlen, 0.0f, grad_weights->as_mut_ptr(), s()), "matrix_scale");
    unwrap(rh_sscal((int64_t)blen, 0.0f, grad_bias->as_mut_ptr(), s()), "row_vector_scale");
  }
  void fused_sgd_step(float l2, float scale, float momentum, float apply) {
    RB_ASSERT(has_backward());
    unwrap(rh_sgd_momentum_step((int64_t)wlen, weights->as_mut_ptr(), grad_weights->as_mut_ptr(),
                                acc_grad_weights->as_mut_ptr(), l2, scale, momentum, apply, 1, s()), "rh_sgd_momentum_step");
    unwrap(rh_sgd_momentum_step((int64_t)blen, bias->as_mut_ptr(), grad_bias->as_mut_ptr(),
                                acc_grad_bias->as_mut_ptr(), l2, scale, momentum, apply, 1, s()), "rh_sgd_momentum_step");
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
  bool buffer(int which, float** ptr, size_t* len) {
    DeviceBuffer<float>* b = nullptr;
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

// ---- Data3dOperator (minimal: u8 staging + cast, or fp32 frames) ------------------------------------------
class Data3dOperator : public InputOperator {
 public:
  Data3dOperator(size_t batch_size, const Data3dOperatorConfig& config, Ctx context)
      : batch_cap_(batch_size), config_(config), context_(context),
        in_buf_h_(batch_size * config.in_dims.len(), 0),
        in_buf_(new DeviceBuffer<uint8_t>(batch_size * config.in_dims.len(), context)),
        out_buf_(new DeviceBuffer<float>(batch_size * config.in_dims.len(), context)) {}
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_buf_; }
  SharedDeviceBuf get_output_deltas() const override { return nullptr; }  // src/operator/mod.rs:632-634
  uint8_t* expose_host_frame_buf(size_t batch_idx) override {
    RB_ASSERT(batch_idx < batch_cap_);
    return in_buf_h_.data() + batch_idx * config_.in_dims.len();
  }
  void load_frames(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    in_buf_->sync_load(in_buf_h_.data(), in_buf_h_.size());
  }
  void load_frames_f32(const float* host, size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    out_buf_->sync_load(host, batch_size * config_.in_dims.len());
    f32_loaded_ = true;
  }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    if (f32_loaded_) return;  // frames were placed in out_buf directly
    const size_t n = batch_size * config_.in_dims.len();
    unwrap(rh_cast_u8_f32(in_buf_->as_ptr(), out_buf_->as_mut_ptr(), n, config_.normalize ? 1.0f / 255.0f : 1.0f,
                          context_->stream()), "cast_bytes");
  }
  void backward(size_t) override {}
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which != 0) return false;
    *ptr = out_buf_->as_mut_ptr();
    *len = out_buf_->len();
    return true;
  }
  const char* kind() const override { return "Data3dOperator"; }

 private:
  size_t batch_cap_;
  Data3dOperatorConfig config_;
  Ctx context_;
  std::vector<uint8_t> in_buf_h_;
  std::unique_ptr<DeviceBuffer<uint8_t>> in_buf_;
  SharedDeviceBuf out_buf_;
  bool f32_loaded_ = false;
};

// ---- AffineOperator -------------------------------------------------------------------------------------
class AffineOperator : public Operator {
 public:
  AffineOperator(size_t batch_size, OpCapability capability, const AffineOperatorConfig& config, const Operator* prev_op,
                 Ctx context)
      : batch_cap_(batch_size), config_(config), context_(context) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("AffineOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.in_channels * batch_size);
    out_act_.reset(new DeviceBuffer<float>(config.out_channels * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(config.out_channels * batch_size, context));
    params_.alloc(config.in_channels * config.out_channels, config.out_channels, backward_enabled(capability), context);
    const int i = (int)config.in_channels, o = (int)config.out_channels, b = (int)batch_size;
    size_t ws = rh_sgemm_workspace_bytes(o, b, i);
    if (backward_enabled(capability)) {
      ws = std::max(ws, rh_sgemm_workspace_bytes(i, o, b));
      ws = std::max(ws, rh_sgemm_workspace_bytes(i, b, o));
    }
    if (ws) workspace_.reset(new DeviceBuffer<uint8_t>(ws, context));
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
    apply_rect_backprop(config_.act_func, out_act_->as_ptr(), config_.out_channels, batch_size, out_delta_->as_mut_ptr(), s);
    // grad_weights(in, out) += in_act(in, B) * out_delta(out, B)^T
    unwrap(rh_sgemm(0, 1, i, o, b, 1.0f, in_act_->as_ptr(), i, out_delta_->as_ptr(), o, 1.0f,
                    params_.grad_weights->as_mut_ptr(), i, ws_ptr(), ws_len(), 0, s), "matrix_prod");
    // grad_bias(1, out) += 1(1, B) * out_delta^T: the column sums of out_delta, without the ones vector
    unwrap(rh_conv2d_bwd_bias(b, o, 1, 1.0f, out_delta_->as_ptr(), 1.0f, params_.grad_bias->as_mut_ptr(), s), "matrix_prod");
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
  void fused_sgd_step(float l2, float scale, float mu, float apply) override { params_.fused_sgd_step(l2, scale, mu, apply); }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    return params_.buffer(which, ptr, len);
  }
  const char* kind() const override { return "AffineOperator"; }

 private:
  void* ws_ptr() { return workspace_ ? workspace_->as_mut_ptr() : nullptr; }
  size_t ws_len() { return workspace_ ? workspace_->len() : 0; }
  size_t batch_cap_;
  AffineOperatorConfig config_;
  Ctx context_;
  SharedDeviceBuf in_act_, in_delta_, out_act_, out_delta_;
  ParamTensors params_;
  std::unique_ptr<DeviceBuffer<uint8_t>> workspace_;
};

// ---- Conv2dOperator -------------------------------------------------------------------------------------
class Conv2dOperator : public Operator {
 public:
  Conv2dOperator(size_t batch_size, OpCapability capability, const Conv2dOperatorConfig& config, const Operator* prev_op,
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
    size_t ws = rh_conv2d_workspace_bytes(&g, RH_CONV_FWD);
    if (backward_enabled(capability)) {
      ws = std::max(ws, rh_conv2d_workspace_bytes(&g, RH_CONV_BWD_FILTER));
      ws = std::max(ws, rh_conv2d_workspace_bytes(&g, RH_CONV_BWD_DATA));
      ws = std::max(ws, rh_conv2d_bwd_bias_workspace_bytes(g.N, g.K, (int)(out_dims_.w * out_dims_.h)));
    }
    workspace_.reset(new DeviceBuffer<uint8_t>(std::max<size_t>(ws, 256), context));
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void init_params(const uint64_t seed[2]) override {
    const size_t fan_in = config_.conv_size * config_.conv_size * config_.in_dims.c;
    params_.init(config_.init_weights, seed, fan_in, config_.out_channels, false, "Conv2dOperator");
  }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_conv_geom g = geom(batch_size);
    rh_stream_t s = context_->stream();
    const bool rect = config_.act_func == ActivationFunction::Rect;
    if (config_.act_func != ActivationFunction::Identity && !rect) panic("unimplemented activation function");
    const int math = opts_.bf16_forward ? RH_MATH_BF16_MFMA_FP32ACC : 0;
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
  void backward(size_t batch_size) override {
    RB_ASSERT(params_.has_backward());
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_conv_geom g = geom(batch_size);
    rh_stream_t s = context_->stream();
    apply_rect_backprop(config_.act_func, out_act_->as_ptr(), out_dims_.len(), batch_size, out_delta_->as_mut_ptr(), s);
    unwrap(rh_conv2d_bwd_filter(&g, 1.0f, in_act_->as_ptr(), out_delta_->as_ptr(), 1.0f, params_.grad_weights->as_mut_ptr(),
                                workspace_->as_mut_ptr(), workspace_->len(), 0, s), "conv2d backward filter");
    unwrap(rh_conv2d_bwd_bias_ws((int)batch_size, (int)out_dims_.c, (int)(out_dims_.w * out_dims_.h), 1.0f,
                                 out_delta_->as_ptr(), 1.0f, params_.grad_bias->as_mut_ptr(), workspace_->as_mut_ptr(),
                                 workspace_->len(), s), "conv2d backward bias");
    if (in_delta_) {
      unwrap(rh_conv2d_bwd_data(&g, 1.0f, params_.weights->as_ptr(), out_delta_->as_ptr(), 0.0f, in_delta_->as_mut_ptr(),
                                workspace_->as_mut_ptr(), workspace_->len(), 0, s), "conv2d backward data");
    }
  }
  void regularize(Regularization reg) override { params_.regularize(reg); }
  void accumulate_grads(float scale, float momentum) override { params_.accumulate_grads(scale, momentum); }
  void update_params(float scale) override { params_.update_params(scale); }
  void update_params2(float g, float u) override { params_.update_params2(g, u); }
  void save_params() override { params_.save_params(); }
  void restore_params() override { params_.restore_params(); }
  void reset() override { params_.reset(); }
  void fused_sgd_step(float l2, float scale, float mu, float apply) override { params_.fused_sgd_step(l2, scale, mu, apply); }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
    if (which == 1) { *ptr = out_delta_->as_mut_ptr(); *len = out_delta_->len(); return true; }
    return params_.buffer(which, ptr, len);
  }
  const char* kind() const override { return "Conv2dOperator"; }

 private:
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
  std::unique_ptr<DeviceBuffer<uint8_t>> workspace_;
};

// ---- Pool2dOperator -------------------------------------------------------------------------------------
class Pool2dOperator : public Operator {
 public:
  Pool2dOperator(size_t batch_size, const Pool2dOperatorConfig& config, const Operator* prev_op, Ctx context)
      : batch_cap_(batch_size), config_(config), context_(context) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("Pool2dOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_act_->len() >= config.in_dims.len() * batch_size);
    out_dims_ = config.get_out_dims();
    out_act_.reset(new DeviceBuffer<float>(out_dims_.len() * batch_size, context));
    out_delta_.reset(new DeviceBuffer<float>(out_dims_.len() * batch_size, context));
    // private arg-max mask: lets backward route deltas without re-scanning the windows
    if (config.pool_op == PoolOperation::Max && in_delta_)
      argmax_.reset(new DeviceBuffer<int32_t>(out_dims_.len() * batch_size, context));
  }
  size_t batch_size() const override { return batch_cap_; }
  SharedDeviceBuf get_output_vars() const override { return out_act_; }
  SharedDeviceBuf get_output_deltas() const override { return out_delta_; }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_pool_geom g = geom(batch_size);
    unwrap(rh_pool2d_fwd(&g, in_act_->as_ptr(), out_act_->as_mut_ptr(), argmax_ ? argmax_->as_mut_ptr() : nullptr,
                         context_->stream()), "pooling forward");
  }
  void backward(size_t batch_size) override {
    if (!in_delta_) return;
    RB_ASSERT(batch_size <= batch_cap_);
    const rh_pool_geom g = geom(batch_size);
    unwrap(rh_pool2d_bwd(&g, in_act_->as_ptr(), out_act_->as_ptr(), out_delta_->as_ptr(), in_delta_->as_mut_ptr(),
                         argmax_ ? argmax_->as_ptr() : nullptr, context_->stream()), "pooling backward");
  }
  bool buffer(int which, float** ptr, size_t* len) override {
    if (which == 0) { *ptr = out_act_->as_mut_ptr(); *len = out_act_->len(); return true; }
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
  std::unique_ptr<DeviceBuffer<int32_t>> argmax_;
};

// ---- SoftmaxKLLossOperator ------------------------------------------------------------------------------
class SoftmaxKLLossOperator : public LossOperator {
 public:
  SoftmaxKLLossOperator(size_t batch_size, const CategoricalLossConfig& loss_config, const Operator* prev_op, Ctx context)
      : batch_cap_(batch_size), loss_config_(loss_config), context_(context),
        label_cats_(batch_size, context), label_cats_h_(batch_size, 0), weights_(batch_size, context),
        weights_h_(batch_size, 0.0f), out_values_(loss_config.num_categories * batch_size, context),
        max_value_(batch_size, context), out_cats_(batch_size, context), out_cats_h_(batch_size, 0),
        out_loss1_(batch_size, context), out_loss_(1, context) {
    RB_ASSERT(prev_op != nullptr);
    in_act_ = prev_op->get_output_vars();
    if (!in_act_) panic("SoftmaxKLLossOperator missing required prev operator output vars");
    in_delta_ = prev_op->get_output_deltas();
    RB_ASSERT(in_delta_ != nullptr);
    RB_ASSERT(in_act_->len() >= loss_config.num_categories * batch_size);
  }
  size_t batch_size() const override { return batch_cap_; }
  void forward(size_t batch_size, OpPhase) override {
    RB_ASSERT(batch_size <= batch_cap_);
    unwrap(rh_softmax_fwd(in_act_->as_ptr(), out_values_.as_mut_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                          context_->stream()), "softmax forward");
  }
  void backward(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
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
    label_cats_.sync_load(label_cats_h_.data(), batch_cap_);
  }
  void stage_weight(size_t batch_idx, float weight) override {
    RB_ASSERT(batch_idx < batch_cap_);
    weights_h_[batch_idx] = weight;
  }
  void load_weights(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    weights_.sync_load(weights_h_.data(), batch_cap_);
  }
  float store_loss(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    rh_stream_t s = context_->stream();
    rembrandt_kernel_batch_map_softmax_kl_loss1(out_values_.as_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                                                label_cats_.as_ptr(), weights_.as_ptr(), 0.0f, out_loss1_.as_mut_ptr(), s);
    unwrap_last("rembrandt_kernel_batch_map_softmax_kl_loss1");
    rembrandt_kernel_batch_blockreduce_sum(out_loss1_.as_ptr(), (int)batch_size, 1, out_loss_.as_mut_ptr(), 0.0f, s);
    unwrap_last("rembrandt_kernel_batch_blockreduce_sum");
    float h = 0.0f;
    out_loss_.sync_store(&h, 1);
    return h;
  }
  void store_output_categories(size_t batch_size) override {
    RB_ASSERT(batch_size <= batch_cap_);
    rembrandt_kernel_batch_blockreduce_argmax(out_values_.as_ptr(), (int)loss_config_.num_categories, (int)batch_size,
                                              max_value_.as_mut_ptr(), out_cats_.as_mut_ptr(), context_->stream());
    unwrap_last("rembrandt_kernel_batch_blockreduce_argmax");
    out_cats_.sync_store(out_cats_h_.data(), batch_cap_);
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
  std::vector<int32_t> out_cats_h_;
  DeviceBuffer<float> out_loss1_, out_loss_;
};

// xorshift128+ used only to derive per-operator seeds from the shared seed
// (Xorshiftplus128Rng in src/operator/worker.rs:361-367; its bit stream is not reproducible here).
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

}  // namespace

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
  input_op_.reset(new Data3dOperator(batch_size, config.input_op.data3d, context));
  const Operator* prev = input_op_.get();
  size_t params_off = 0;
  for (const auto& c : config.hidden_ops) {
    std::unique_ptr<Operator> op;
    switch (c.kind) {
      case OperatorConfig::Affine: op.reset(new AffineOperator(batch_size, capability, c.affine, prev, context)); break;
      case OperatorConfig::Conv2d: op.reset(new Conv2dOperator(batch_size, capability, c.conv2d, prev, context, opts)); break;
      case OperatorConfig::Pool2d: op.reset(new Pool2dOperator(batch_size, c.pool2d, prev, context)); break;
      default: panic("SequentialOperatorWorker: not a hidden operator");
    }
    params_off += c.params_len();
    hidden_ops_.push_back(std::move(op));
    prev = hidden_ops_.back().get();
  }
  RB_ASSERT(params_off == config.params_len());  // src/operator/worker.rs:289
  loss_op_.reset(new SoftmaxKLLossOperator(batch_size, config.loss_op.loss, prev, context));
  context_->sync();
}

LossOperator* SequentialOperatorWorker::loss_operator(size_t rank) {
  RB_ASSERT(rank == 0);
  return loss_op_.get();
}

void SequentialOperatorWorker::init_params(const uint64_t shared_seed[2]) {
  Xorshiftplus128 rng(shared_seed);
  for (auto& op : hidden_ops_) {
    const uint64_t op_seed[2] = {rng.next_u64(), rng.next_u64()};
    op->init_params(op_seed);
  }
}
void SequentialOperatorWorker::forward(size_t batch_size, OpPhase phase) {
  input_op_->forward(batch_size, phase);
  for (auto& op : hidden_ops_) op->forward(batch_size, phase);
  loss_op_->forward(batch_size, phase);
}
void SequentialOperatorWorker::backward(size_t batch_size) {
  loss_op_->backward(batch_size);
  for (auto it = hidden_ops_.rbegin(); it != hidden_ops_.rend(); ++it) (*it)->backward(batch_size);
}
void SequentialOperatorWorker::regularize(Regularization reg) { for (auto& op : hidden_ops_) op->regularize(reg); }
void SequentialOperatorWorker::accumulate_grads(float scale, float momentum) { for (auto& op : hidden_ops_) op->accumulate_grads(scale, momentum); }
void SequentialOperatorWorker::update_params(float scale) { for (auto& op : hidden_ops_) op->update_params(scale); }
void SequentialOperatorWorker::update_params2(float g, float u) { for (auto& op : hidden_ops_) op->update_params2(g, u); }
void SequentialOperatorWorker::save_params() { for (auto& op : hidden_ops_) op->save_params(); }
void SequentialOperatorWorker::restore_params() { for (auto& op : hidden_ops_) op->restore_params(); }
void SequentialOperatorWorker::reset() { for (auto& op : hidden_ops_) op->reset(); }
void SequentialOperatorWorker::fused_sgd_step(float l2, float scale, float mu, float apply) {
  for (auto& op : hidden_ops_) op->fused_sgd_step(l2, scale, mu, apply);
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

void SgdOpt::step(Operator* op, bool fused) {
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
  if (k == Momentum::UpdateNesterov) op->update_params(mu);
}

}  // namespace rembrandt
