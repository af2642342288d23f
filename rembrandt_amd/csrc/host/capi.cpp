// C ABI of the operator / graph / optimizer layer (include/rembrandt_operator.h).
#include <cstdio>
#include <memory>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <tuple>
#include <vector>
#include <algorithm>

#include "../../../include/rembrandt_operator.h"
#include "data_source.hpp"
#include "model_config.hpp"
#include "operator.hpp"

using namespace rembrandt;

struct rho_config { SequentialOperatorConfig cfg; };
// What makes two train steps the same sequence of launches with the same arguments.
struct StepKey {
  size_t batch;
  int fused, momentum_kind;
  uint32_t step_size_bits, l2_bits, mu_bits;
  bool first_iter;  // the Nesterov un-apply is skipped at iteration 0
  int input_mode;   // which loader filled the input frames: the input operator's forward launches differ
  std::vector<char> grad_state;  // which operators' gradient buffers stand for zeros: their backward passes overwrite (beta = 0)
  bool operator<(const StepKey& o) const {
    return std::tie(batch, fused, momentum_kind, step_size_bits, l2_bits, mu_bits, first_iter, input_mode, grad_state) <
           std::tie(o.batch, o.fused, o.momentum_kind, o.step_size_bits, o.l2_bits, o.mu_bits, o.first_iter, o.input_mode,
                    o.grad_state);
  }
};
// A schedule whose step size changes every iteration (Inverse) never repeats a key: neither set may grow with it.
constexpr size_t kMaxSeenSteps = 64, kMaxStepGraphs = 16;

struct rho_worker {
  std::shared_ptr<DeviceContext> ctx;
  std::unique_ptr<SequentialOperatorWorker> worker;
  bool graph_steps = false;
  bool fuse_epilogue = false;                // also: the loss operator's one-launch form inside rho_sgd_train_batch
  int64_t graph_launches = 0;                // steps that ran as a graph launch
  struct RecordedStep {
    rh_graph* graph;
    std::vector<char> grad_state_after;      // host-side state the recorded calls left behind (restored after a replay)
  };
  std::map<StepKey, RecordedStep> step_graphs;  // recorded steps
  std::set<StepKey> seen_steps;              // combinations that ran once launch by launch
  void drop_graphs() {
    for (auto& kv : step_graphs) (void)rh_graph_destroy(kv.second.graph);
    step_graphs.clear();
    seen_steps.clear();
  }
  ~rho_worker() {
    if (ctx) (void)rh_ctx_sync(ctx->raw());
    drop_graphs();
  }
};
struct rho_sgd { std::unique_ptr<SgdOpt> opt; };
struct rho_dataset { std::unique_ptr<DataSource> src; };

static thread_local std::string g_message;

#define RHO_TRY(...)                                    \
  try { __VA_ARGS__; return 0; }                        \
  catch (const std::exception& e) { g_message = e.what(); return RHO_E_PANIC; } \
  catch (...) { g_message = "unknown exception"; return RHO_E_PANIC; }

#define RHO_REQ(cond) do { if (!(cond)) panic(std::string("invalid argument: ") + #cond); } while (0)

static ActivationFunction act_of(int a) {
  switch (a) {
    case RHO_ACT_IDENTITY: return ActivationFunction::Identity;
    case RHO_ACT_RECT: return ActivationFunction::Rect;
    case RHO_ACT_LOGISTIC: return ActivationFunction::Logistic;
    case RHO_ACT_TANH: return ActivationFunction::Tanh;
  }
  panic("unknown activation function");
}
static ParamsInit init_of(int kind, float v) {
  switch (kind) {
    case RHO_INIT_DISABLED: return ParamsInit::MakeDisabled();
    case RHO_INIT_UNIFORM: return ParamsInit::MakeUniform(v);
    case RHO_INIT_NORMAL: return ParamsInit::MakeNormal(v);
    case RHO_INIT_XAVIER: return ParamsInit::MakeXavier();
    case RHO_INIT_KAIMING_FWD: return ParamsInit::MakeKaimingFwd();
  }
  panic("unknown params init");
}

static Operator* op_at(rho_worker* w, int32_t idx) {
  RHO_REQ(w && w->worker);
  const int32_t n = (int32_t)w->worker->hidden_count();
  if (idx == -1) return w->worker->input_operator();
  if (idx == n) return w->worker->loss_operator(0);
  RHO_REQ(idx >= 0 && idx < n);
  return w->worker->hidden_operator((size_t)idx);
}

extern "C" {

const char* rho_last_message(void) { return g_message.c_str(); }

int rho_config_new(rho_config** out) { RHO_TRY({ RHO_REQ(out); *out = new rho_config(); }) }
int rho_config_free(rho_config* cfg) { RHO_TRY({ delete cfg; }) }

int rho_config_data3d(rho_config* cfg, int32_t w, int32_t h, int32_t c, int normalize) {
  RHO_TRY({
    RHO_REQ(cfg && w > 0 && h > 0 && c > 0);
    Data3dOperatorConfig d = {{(size_t)w, (size_t)h, (size_t)c}, normalize != 0};
    cfg->cfg.data3d(d);
  })
}
static Data3dOperatorConfig& input_cfg(rho_config* cfg) {
  RHO_REQ(cfg && cfg->cfg.has_input);
  return cfg->cfg.input_op.data3d;
}
int rho_config_data3d_crop(rho_config* cfg, int32_t crop_width, int32_t crop_height) {
  RHO_TRY({
    RHO_REQ(crop_width > 0 && crop_height > 0);
    Data3dPreproc p;
    p.kind = Data3dPreproc::Crop;
    p.crop_width = (size_t)crop_width;
    p.crop_height = (size_t)crop_height;
    input_cfg(cfg).preprocs.push_back(p);
    (void)input_cfg(cfg).get_out_dims();
  })
}
int rho_config_data3d_flip_x(rho_config* cfg) {
  RHO_TRY({
    Data3dPreproc p;
    p.kind = Data3dPreproc::FlipX;
    input_cfg(cfg).preprocs.push_back(p);
  })
}
int rho_config_data3d_subtract_mean(rho_config* cfg, const float* mean, int64_t len) {
  RHO_TRY({
    RHO_REQ(mean && len == (int64_t)input_cfg(cfg).in_dims.len());
    Data3dPreproc p;
    p.kind = Data3dPreproc::SubtractElemwiseMean;
    p.mean_values.assign(mean, mean + len);
    input_cfg(cfg).preprocs.push_back(p);
  })
}
int rho_config_data3d_subtract_mean_file(rho_config* cfg, const char* mean_path) {
  RHO_TRY({
    RHO_REQ(mean_path && *mean_path);
    Data3dPreproc p;
    p.kind = Data3dPreproc::SubtractElemwiseMean;
    p.mean_path = mean_path;
    input_cfg(cfg).preprocs.push_back(p);
  })
}
int rho_config_data3d_pca_lighting_noise(rho_config* cfg, const float* singular_vecs9, const float* singular_vals3, float std_dev) {
  RHO_TRY({
    RHO_REQ(singular_vecs9 && singular_vals3 && std_dev >= 0.0f);
    Data3dPreproc p;
    p.kind = Data3dPreproc::AddPixelwisePCALightingNoise;
    for (int i = 0; i < 3; ++i) {
      for (int j = 0; j < 3; ++j) p.singular_vecs[i][j] = singular_vecs9[i * 3 + j];
      p.singular_vals[i] = singular_vals3[i];
    }
    p.std_dev = std_dev;
    input_cfg(cfg).preprocs.push_back(p);
  })
}
int rho_config_dropout(rho_config* cfg, int32_t channels, float drop_ratio) {
  RHO_TRY({
    RHO_REQ(cfg && channels > 0 && drop_ratio >= 0.0f && drop_ratio <= 1.0f);
    DropoutOperatorConfig d = {(size_t)channels, drop_ratio};
    cfg->cfg.dropout(d);
  })
}
int rho_config_local_res_norm(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t cross_size, float scale,
                              float power, float min_div) {
  RHO_TRY({
    RHO_REQ(cfg && in_w > 0 && in_h > 0 && in_c > 0 && cross_size > 0 && min_div > 0.0f);
    LocalResNormOperatorConfig l = {{(size_t)in_w, (size_t)in_h, (size_t)in_c}, (size_t)cross_size, scale, power, min_div};
    cfg->cfg.local_res_norm(l);
  })
}
int rho_config_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t conv_size, int32_t conv_stride,
                      int32_t conv_pad, int32_t out_channels, int act_func, int init_kind, float init_value) {
  RHO_TRY({
    RHO_REQ(cfg && in_w > 0 && in_h > 0 && in_c > 0 && conv_size > 0 && conv_stride > 0 && conv_pad >= 0 && out_channels > 0);
    Conv2dOperatorConfig c = {{(size_t)in_w, (size_t)in_h, (size_t)in_c}, (size_t)conv_size, (size_t)conv_stride,
                              (size_t)conv_pad, (size_t)out_channels, act_of(act_func), init_of(init_kind, init_value)};
    cfg->cfg.conv2d(c);
  })
}
static BNormMovingAverage mov_avg_of(int kind, double ema_factor) {
  if (kind == RHO_BNORM_CUMULATIVE) return BNormMovingAverage::MakeCumulative();
  if (kind != RHO_BNORM_EXPONENTIAL || !(ema_factor >= 0.0 && ema_factor <= 1.0)) panic("unknown batch norm moving average");
  return BNormMovingAverage::MakeExponential(ema_factor);
}
int rho_config_bnorm_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t conv_size, int32_t conv_stride,
                            int32_t conv_pad, int32_t out_channels, int mov_avg_kind, double ema_factor, double epsilon,
                            int act_func, int init_kind, float init_value) {
  RHO_TRY({
    RHO_REQ(cfg && in_w > 0 && in_h > 0 && in_c > 0 && conv_size > 0 && conv_stride > 0 && conv_pad >= 0 && out_channels > 0);
    RHO_REQ(epsilon > 0.0);
    BNormConv2dOperatorConfig c = {{(size_t)in_w, (size_t)in_h, (size_t)in_c}, (size_t)conv_size, (size_t)conv_stride,
                                   (size_t)conv_pad, (size_t)out_channels, mov_avg_of(mov_avg_kind, ema_factor), epsilon,
                                   act_of(act_func), init_of(init_kind, init_value)};
    cfg->cfg.bnorm_conv2d(c);
  })
}
int rho_config_stack_res_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int mov_avg_kind, double ema_factor,
                                double epsilon, int act_func, int init_kind, float init_value) {
  RHO_TRY({
    RHO_REQ(cfg && in_w > 0 && in_h > 0 && in_c > 0 && epsilon > 0.0);
    StackResConv2dOperatorConfig c = {{(size_t)in_w, (size_t)in_h, (size_t)in_c}, mov_avg_of(mov_avg_kind, ema_factor), epsilon,
                                      act_of(act_func), init_of(init_kind, init_value)};
    cfg->cfg.stack_res_conv2d(c);
  })
}
int rho_config_proj_stack_res_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t out_w, int32_t out_h,
                                     int32_t out_c, int mov_avg_kind, double ema_factor, double epsilon, int act_func,
                                     int init_kind, float init_value) {
  RHO_TRY({
    RHO_REQ(cfg && in_w > 0 && in_h > 0 && in_c > 0 && out_w > 0 && out_h > 0 && out_c > 0 && epsilon > 0.0);
    RHO_REQ((in_w == out_w && in_h == out_h) || (in_w == 2 * out_w && in_h == 2 * out_h));
    ProjStackResConv2dOperatorConfig c = {{(size_t)in_w, (size_t)in_h, (size_t)in_c}, {(size_t)out_w, (size_t)out_h, (size_t)out_c},
                                          mov_avg_of(mov_avg_kind, ema_factor), epsilon, act_of(act_func),
                                          init_of(init_kind, init_value)};
    cfg->cfg.proj_stack_res_conv2d(c);
  })
}
int rho_config_affine(rho_config* cfg, int32_t in_channels, int32_t out_channels, int act_func, int init_kind, float init_value) {
  RHO_TRY({
    RHO_REQ(cfg && in_channels > 0 && out_channels > 0);
    AffineOperatorConfig a = {(size_t)in_channels, (size_t)out_channels, act_of(act_func), init_of(init_kind, init_value)};
    cfg->cfg.affine(a);
  })
}
int rho_config_pool2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t pool_size, int32_t pool_stride,
                      int32_t pool_pad, int pool_op, int ceil_mode) {
  RHO_TRY({
    RHO_REQ(cfg && in_w > 0 && in_h > 0 && in_c > 0 && pool_size > 0 && pool_stride > 0 && pool_pad >= 0);
    RHO_REQ(pool_op == RHO_POOL_MAX || pool_op == RHO_POOL_AVERAGE);
    Pool2dOperatorConfig p = {{(size_t)in_w, (size_t)in_h, (size_t)in_c}, (size_t)pool_size, (size_t)pool_stride,
                              (size_t)pool_pad, pool_op == RHO_POOL_MAX ? PoolOperation::Max : PoolOperation::Average,
                              ActivationFunction::Identity, ceil_mode != 0};
    cfg->cfg.pool2d(p);
  })
}
int rho_config_softmax_kl_loss(rho_config* cfg, int32_t num_categories) {
  RHO_TRY({
    RHO_REQ(cfg && num_categories > 0);
    CategoricalLossConfig l = {(size_t)num_categories};
    cfg->cfg.softmax_kl_loss(l);
  })
}
int rho_config_params_len(const rho_config* cfg, int64_t* out) {
  RHO_TRY({ RHO_REQ(cfg && out); *out = (int64_t)cfg->cfg.params_len(); })
}
int rho_config_from_model_file(const char* path, rho_config** out) {
  RHO_TRY({
    RHO_REQ(path && out);
    std::unique_ptr<rho_config> c(new rho_config());
    c->cfg = ModelConfigFile::open(path).to_sequential_config();
    *out = c.release();
  })
}

int rho_worker_new(const rho_config* cfg, int32_t batch_size, int capability, uint64_t seed0, uint64_t seed1, int device,
                   int exec_flags, rho_worker** out) {
  RHO_TRY({
    RHO_REQ(cfg && out && batch_size > 0);
    std::unique_ptr<rho_worker> w(new rho_worker());
    w->ctx = std::make_shared<DeviceContext>(device);
    const uint64_t seed[2] = {seed0, seed1};
    ExecOptions opts;
    opts.fuse_epilogue = (exec_flags & RHO_EXEC_FUSE_EPILOGUE) != 0;
    opts.bf16_forward = (exec_flags & RHO_EXEC_BF16_FORWARD) != 0;
    opts.overlap_backward = (exec_flags & RHO_EXEC_OVERLAP_BACKWARD) != 0;
    opts.graph_steps = (exec_flags & RHO_EXEC_GRAPH_STEPS) != 0;
    opts.fuse_tail = (exec_flags & RHO_EXEC_SEPARATE_TAIL) == 0;
    opts.winograd = (exec_flags & RHO_EXEC_DIRECT_CONV) == 0;
    w->graph_steps = opts.graph_steps;
    w->fuse_epilogue = opts.fuse_epilogue;
    w->worker.reset(new SequentialOperatorWorker(cfg->cfg, (size_t)batch_size,
                                                 capability == RHO_CAP_FORWARD ? OpCapability::Forward : OpCapability::Backward,
                                                 seed, w->ctx, opts));
    *out = w.release();
  })
}
int rho_worker_free(rho_worker* w) { RHO_TRY({ delete w; }) }
int rho_worker_set_overlap_backward(rho_worker* w, int on) {
  RHO_TRY({
    RHO_REQ(w);
    w->ctx->sync();
    w->drop_graphs();  // recorded steps carry the old placement
    w->worker->set_overlap_backward(on != 0);
  })
}
int rho_worker_graph_launches(rho_worker* w, int64_t* out) { RHO_TRY({ RHO_REQ(w && out); *out = w->graph_launches; }) }
int rho_worker_hidden_count(rho_worker* w, int32_t* out) { RHO_TRY({ RHO_REQ(w && out); *out = (int32_t)w->worker->hidden_count(); }) }
int rho_worker_op_kind(rho_worker* w, int32_t hidden_idx, const char** out) { RHO_TRY({ RHO_REQ(out); *out = op_at(w, hidden_idx)->kind(); }) }
void* rho_worker_stream(rho_worker* w) { return w ? w->ctx->stream() : nullptr; }
int rho_worker_sync(rho_worker* w) { RHO_TRY({ RHO_REQ(w); w->ctx->sync(); }) }
int rho_worker_init_params(rho_worker* w, uint64_t seed0, uint64_t seed1) {
  RHO_TRY({ RHO_REQ(w); const uint64_t s[2] = {seed0, seed1}; w->worker->init_params(s); })
}
int rho_worker_expose_host_frame_buf(rho_worker* w, int32_t batch_idx, uint8_t** out) {
  RHO_TRY({ RHO_REQ(w && out && batch_idx >= 0); *out = w->worker->input_operator()->expose_host_frame_buf((size_t)batch_idx); })
}
int rho_worker_load_frames(rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->input_operator()->load_frames((size_t)batch_size); })
}
int rho_worker_load_frames_f32(rho_worker* w, const float* host, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && host && batch_size >= 0); w->worker->input_operator()->load_frames_f32(host, (size_t)batch_size); })
}
int rho_worker_input_out_dims(rho_worker* w, int32_t* out_w, int32_t* out_h, int32_t* out_c) {
  RHO_TRY({
    RHO_REQ(w && out_w && out_h && out_c);
    const Dims3 d = w->worker->input_operator()->out_dims();
    *out_w = (int32_t)d.w; *out_h = (int32_t)d.h; *out_c = (int32_t)d.c;
  })
}
int rho_worker_last_preproc_draws(rho_worker* w, int32_t* crop_off_w, int32_t* crop_off_h, int* flipped, float* alphas,
                                  int64_t alphas_cap, int64_t* alphas_len) {
  RHO_TRY({
    RHO_REQ(w);
    size_t ow = 0, oh = 0;
    bool fl = false;
    std::vector<float> a;
    w->worker->input_operator()->last_preproc_draws(&ow, &oh, &fl, &a);
    if (crop_off_w) *crop_off_w = (int32_t)ow;
    if (crop_off_h) *crop_off_h = (int32_t)oh;
    if (flipped) *flipped = fl ? 1 : 0;
    if (alphas_len) *alphas_len = (int64_t)a.size();
    if (alphas) {
      RHO_REQ(alphas_cap >= (int64_t)a.size());
      for (size_t i = 0; i < a.size(); ++i) alphas[i] = a[i];
    }
  })
}
int rho_worker_dropout_stream(rho_worker* w, int32_t hidden_idx, uint64_t* seed, uint64_t* stream_id, uint64_t* first) {
  RHO_TRY({
    RHO_REQ(w && seed && stream_id && first && hidden_idx >= 0 && (size_t)hidden_idx < w->worker->hidden_count());
    if (!w->worker->dropout_stream((size_t)hidden_idx, seed, stream_id, first)) panic("not a DropoutOperator");
  })
}
static int copy_blob(const std::vector<uint8_t>& blob, uint8_t* buf, size_t cap, size_t* needed) {
  if (needed) *needed = blob.size();
  if (buf) {
    if (cap < blob.size()) panic("blob buffer too small");
    std::copy(blob.begin(), blob.end(), buf);
  }
  return 0;
}
int rho_worker_encode_params(rho_worker* w, uint8_t* buf, size_t cap, size_t* needed) {
  RHO_TRY({ RHO_REQ(w); std::vector<uint8_t> b; w->worker->encode_params(b); copy_blob(b, buf, cap, needed); })
}
int rho_worker_decode_params(rho_worker* w, const uint8_t* blob, size_t len, size_t* consumed) {
  RHO_TRY({ RHO_REQ(w && blob); const size_t n = w->worker->decode_params(blob, len); if (consumed) *consumed = n; })
}
int rho_worker_encode_state(rho_worker* w, uint8_t* buf, size_t cap, size_t* needed) {
  RHO_TRY({ RHO_REQ(w); std::vector<uint8_t> b; w->worker->encode_state(b); copy_blob(b, buf, cap, needed); })
}
int rho_worker_decode_state(rho_worker* w, const uint8_t* blob, size_t len, size_t* consumed) {
  RHO_TRY({ RHO_REQ(w && blob); const size_t n = w->worker->decode_state(blob, len); if (consumed) *consumed = n; })
}
int rho_worker_checkpoint_params(rho_worker* w, int64_t t, const char* prefix) {
  RHO_TRY({ RHO_REQ(w && prefix && t >= 0); w->worker->checkpoint_params((size_t)t, prefix); })
}
int rho_worker_checkpoint_state(rho_worker* w, const char* prefix) {
  RHO_TRY({ RHO_REQ(w && prefix); w->worker->checkpoint_state(prefix); })
}
int rho_worker_can_rollback(rho_worker* w, const char* prefix, int64_t* t_or_minus1) {
  RHO_TRY({
    RHO_REQ(w && prefix && t_or_minus1);
    size_t t = 0;
    *t_or_minus1 = w->worker->can_rollback(prefix, &t) ? (int64_t)t : -1;
  })
}
int rho_worker_rollback_params(rho_worker* w, int64_t t_or_minus1, const char* prefix) {
  RHO_TRY({
    RHO_REQ(w && prefix);
    const size_t t = (size_t)t_or_minus1;
    w->worker->rollback_params(t_or_minus1 >= 0 ? &t : nullptr, prefix);
  })
}
int rho_worker_rollback_state(rho_worker* w, const char* prefix) {
  RHO_TRY({ RHO_REQ(w && prefix); w->worker->rollback_state(prefix); })
}
int rho_worker_stage_label(rho_worker* w, int32_t batch_idx, int32_t category) {
  RHO_TRY({ RHO_REQ(w && batch_idx >= 0); w->worker->loss_operator(0)->stage_label((size_t)batch_idx, category); })
}
int rho_worker_load_labels(rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->loss_operator(0)->load_labels((size_t)batch_size); })
}
int rho_worker_stage_weight(rho_worker* w, int32_t batch_idx, float weight) {
  RHO_TRY({ RHO_REQ(w && batch_idx >= 0); w->worker->loss_operator(0)->stage_weight((size_t)batch_idx, weight); })
}
int rho_worker_load_weights(rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->loss_operator(0)->load_weights((size_t)batch_size); })
}
int rho_worker_store_loss(rho_worker* w, int32_t batch_size, float* out) {
  RHO_TRY({ RHO_REQ(w && out && batch_size >= 0); *out = w->worker->loss_operator(0)->store_loss((size_t)batch_size); })
}
int rho_worker_store_output_categories(rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->loss_operator(0)->store_output_categories((size_t)batch_size); })
}
int rho_worker_get_output_categories(rho_worker* w, int32_t batch_size, int32_t* host_out) {
  RHO_TRY({
    RHO_REQ(w && host_out && batch_size >= 0 && (size_t)batch_size <= w->worker->batch_size());
    const int32_t* c = w->worker->loss_operator(0)->get_output_categories((size_t)batch_size);
    for (int32_t i = 0; i < batch_size; ++i) host_out[i] = c[i];
  })
}
int rho_worker_accuracy_count(rho_worker* w, int32_t batch_size, int32_t* out) {
  RHO_TRY({ RHO_REQ(w && out && batch_size >= 0); *out = (int32_t)w->worker->loss_operator(0)->accuracy_count((size_t)batch_size); })
}
int rho_worker_forward(rho_worker* w, int32_t batch_size, int training, int64_t t) {
  RHO_TRY({
    RHO_REQ(w && batch_size >= 0);
    w->worker->forward((size_t)batch_size, training ? OpPhase::Training((size_t)t) : OpPhase::Inference());
  })
}
int rho_worker_backward(rho_worker* w, int32_t batch_size) { RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->backward((size_t)batch_size); }) }
int rho_worker_regularize(rho_worker* w, float l2) { RHO_TRY({ RHO_REQ(w); w->worker->regularize(Regularization::L2(l2)); }) }
int rho_worker_accumulate_grads(rho_worker* w, float scale, float momentum) { RHO_TRY({ RHO_REQ(w); w->worker->accumulate_grads(scale, momentum); }) }
int rho_worker_update_params(rho_worker* w, float scale) { RHO_TRY({ RHO_REQ(w); w->worker->update_params(scale); }) }
int rho_worker_update_params2(rho_worker* w, float g, float u) { RHO_TRY({ RHO_REQ(w); w->worker->update_params2(g, u); }) }
int rho_worker_save_params(rho_worker* w) { RHO_TRY({ RHO_REQ(w); w->worker->save_params(); }) }
int rho_worker_restore_params(rho_worker* w) { RHO_TRY({ RHO_REQ(w); w->worker->restore_params(); }) }
int rho_worker_reset(rho_worker* w) { RHO_TRY({ RHO_REQ(w); w->worker->reset(); }) }

int rho_worker_backward_scaled(rho_worker* w, int32_t batch_size, float scale) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->backward_scaled((size_t)batch_size, scale); })
}
int rho_worker_descend(rho_worker* w, float scale, float l2, int fused) { RHO_TRY({ RHO_REQ(w); w->worker->descend(scale, l2, fused != 0); }) }
int rho_worker_reset_gradients(rho_worker* w, float momentum) { RHO_TRY({ RHO_REQ(w); w->worker->reset_gradients(momentum); }) }
int rho_worker_reset_loss(rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->loss_operator(0)->reset_loss((size_t)batch_size); })
}
int rho_worker_accumulate_loss(rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(w && batch_size >= 0); w->worker->loss_operator(0)->accumulate_loss((size_t)batch_size); })
}
int rho_worker_store_accumulated_loss(rho_worker* w, float* out) {
  RHO_TRY({ RHO_REQ(w && out); *out = w->worker->loss_operator(0)->store_accumulated_loss(); })
}

struct rho_sgd2 {
  std::unique_ptr<SgdOptimization> opt;
};
int rho_sgd2_new(int32_t minibatch_size, int step_kind, const float* steps, const int64_t* step_iters, float momentum,
                 float l2_reg_coef, rho_sgd2** out) {
  RHO_TRY({
    RHO_REQ(out && steps && minibatch_size > 0 && step_kind >= 0 && step_kind <= RHO_STEP_INVERSE);
    SgdOpt2Config c = SgdOpt2Config();
    c.minibatch_size = (size_t)minibatch_size;
    c.step_size.kind = (StepSizeSchedule::Kind)step_kind;
    for (int i = 0; i < 5; ++i) {
      c.step_size.step[i] = steps[i];
      c.step_size.iters[i] = step_iters ? (size_t)step_iters[i] : 0;
    }
    c.momentum = momentum;
    c.l2_reg_coef = l2_reg_coef;
    std::unique_ptr<rho_sgd2> s(new rho_sgd2());
    s->opt.reset(new SgdOptimization(c));
    *out = s.release();
  })
}
int rho_sgd2_free(rho_sgd2* s) { RHO_TRY({ delete s; }) }
int rho_sgd2_begin(rho_sgd2* s, rho_worker* w) { RHO_TRY({ RHO_REQ(s && w); s->opt->begin(w->worker.get()); }) }
int rho_sgd2_batch(rho_sgd2* s, rho_worker* w, int32_t batch_size) {
  RHO_TRY({ RHO_REQ(s && w && batch_size > 0); s->opt->batch(w->worker.get(), (size_t)batch_size); })
}
int rho_sgd2_end_minibatch(rho_sgd2* s, rho_worker* w, int fused) {
  RHO_TRY({ RHO_REQ(s && w); s->opt->end_minibatch(w->worker.get(), fused != 0); })
}
int rho_sgd2_iter_counter(rho_sgd2* s, int64_t* out) { RHO_TRY({ RHO_REQ(s && out); *out = (int64_t)s->opt->iter_counter(); }) }

int rho_worker_buffer(rho_worker* w, int32_t hidden_idx, int which, float** dptr, int64_t* len) {
  RHO_TRY({
    RHO_REQ(dptr && len);
    size_t n = 0;
    RHO_REQ(w);
    w->worker->settle();
    if (!op_at(w, hidden_idx)->buffer(which, dptr, &n)) panic("operator has no such buffer");
    *len = (int64_t)n;
  })
}
int rho_worker_read_buffer(rho_worker* w, int32_t hidden_idx, int which, float* host, int64_t len) {
  RHO_TRY({
    RHO_REQ(w && host && len >= 0);
    w->worker->settle();
    float* d = nullptr;
    size_t n = 0;
    if (!op_at(w, hidden_idx)->buffer(which, &d, &n)) panic("operator has no such buffer");
    RHO_REQ((size_t)len <= n);
    unwrap(rh_store_sync(w->ctx->raw(), host, d, (size_t)len * sizeof(float)), "sync_store");
  })
}
int rho_worker_write_buffer(rho_worker* w, int32_t hidden_idx, int which, const float* host, int64_t len) {
  RHO_TRY({
    RHO_REQ(w && host && len >= 0);
    w->worker->settle();
    float* d = nullptr;
    size_t n = 0;
    if (!op_at(w, hidden_idx)->buffer(which, &d, &n)) panic("operator has no such buffer");
    RHO_REQ((size_t)len <= n);
    unwrap(rh_load_sync(w->ctx->raw(), d, host, (size_t)len * sizeof(float)), "sync_load");
  })
}

int rho_sgd_new(int32_t minibatch_size, int step_kind, const float* steps, const int64_t* step_iters, int momentum_kind,
                float mu, float l2_reg_coef, rho_sgd** out) {
  RHO_TRY({
    RHO_REQ(out && steps && minibatch_size > 0 && step_kind >= 0 && step_kind <= RHO_STEP_INVERSE);
    RHO_REQ(momentum_kind >= 0 && momentum_kind <= RHO_MOM_GRADIENT_NESTEROV);
    SgdOptConfig c = SgdOptConfig();
    c.minibatch_size = (size_t)minibatch_size;
    c.step_size.kind = (StepSizeSchedule::Kind)step_kind;
    for (int i = 0; i < 5; ++i) {
      c.step_size.step[i] = steps[i];
      c.step_size.iters[i] = step_iters ? (size_t)step_iters[i] : 0;
    }
    c.momentum.kind = (Momentum::Kind)momentum_kind;
    c.momentum.mu = mu;
    c.l2_reg_coef = l2_reg_coef;
    std::unique_ptr<rho_sgd> s(new rho_sgd());
    s->opt.reset(new SgdOpt(c));
    *out = s.release();
  })
}
int rho_sgd_free(rho_sgd* s) { RHO_TRY({ delete s; }) }
int rho_sgd_begin(rho_sgd* s, rho_worker* w) { RHO_TRY({ RHO_REQ(s && w); s->opt->begin(w->worker.get()); }) }
int rho_sgd_step(rho_sgd* s, rho_worker* w, int fused) { RHO_TRY({ RHO_REQ(s && w); s->opt->step(w->worker.get(), fused != 0); }) }
int rho_sgd_set_iter_counter(rho_sgd* s, int64_t t) { RHO_TRY({ RHO_REQ(s && t >= 0); s->opt->set_iter_counter((size_t)t); }) }
int rho_sgd_iter_counter(rho_sgd* s, int64_t* out) { RHO_TRY({ RHO_REQ(s && out); *out = (int64_t)s->opt->iter_counter(); }) }
int rho_sgd_step_size_at(rho_sgd* s, int64_t t, float* out) {
  RHO_TRY({ RHO_REQ(s && out && t >= 0); *out = s->opt->config().step_size.at_iter((size_t)t); })
}
static uint32_t float_bits(float v) {
  uint32_t u;
  std::memcpy(&u, &v, sizeof u);
  return u;
}

int rho_sgd_train_batch(rho_sgd* s, rho_worker* w, int32_t batch_size, int fused, float* loss_out, int32_t* correct_out) {
  RHO_TRY({
    RHO_REQ(s && w && batch_size > 0);
    SequentialOperatorWorker* op = w->worker.get();
    const size_t b = (size_t)batch_size;
    const size_t t = s->opt->iter_counter();
    const OpPhase phase = OpPhase::Training(t);
    // With fused epilogues the loss operator produces probabilities, categories, loss and delta in one launch of its
    // forward(); the three calls below that ask for them then launch nothing.
    // (so does the classifier tail, where the chain ends in one: two launches for its ten)
    struct Armed {
      SequentialOperatorWorker* o;
      Armed(SequentialOperatorWorker* o_, bool on) : o(on && o_->arm_train_step(true) ? o_ : nullptr) {}
      ~Armed() { if (o) o->arm_train_step(false); }
    } armed(op, w->fuse_epilogue);
    // forward -> arg-max and loss kernels -> backward -> update are all enqueued before the two read-backs, so
    // the GPU works through the step without waiting for the host (same results as the reference's order:
    // store_output_categories, store_loss, backward; nothing in between writes what they read)
    auto enqueue_step = [&]() {
      op->forward(b, phase);
      op->loss_operator(0)->enqueue_output_categories(b);
      op->loss_operator(0)->enqueue_loss(b);
      op->backward(b);
      s->opt->step(op, fused != 0);
    };
    bool done = false;
    if (w->graph_steps && !rh_profile_enabled() && op->graph_safe(phase)) {
      const SgdOptConfig& c = s->opt->config();
      const StepKey key = {b, fused != 0 ? 1 : 0, (int)c.momentum.kind, float_bits(c.step_size.at_iter(t)),
                           float_bits(c.l2_reg_coef), float_bits(c.momentum.mu), t == 0,
                           op->input_operator()->input_mode(), op->grad_state()};
      auto it = w->step_graphs.find(key);
      if (it != w->step_graphs.end()) {
        w->ctx->launch(it->second.graph);
        s->opt->set_iter_counter(t + 1);  // what step() does on the host
        op->set_grad_state(it->second.grad_state_after);
        w->graph_launches += 1;
        done = true;
      } else if (w->seen_steps.count(key) && w->step_graphs.size() < kMaxStepGraphs) {
        // second time: record.  (The first time ran launch by launch, which also created everything that is made on
        // first use: the second stream, kernel attributes.)
        op->settle();
        w->ctx->begin_capture();
        try {
          enqueue_step();
          op->settle();  // updates issued on the second stream rejoin the recording
        } catch (...) {
          w->ctx->abort_capture();
          op->forget_pending();
          s->opt->set_iter_counter(t);
          op->set_grad_state(key.grad_state);
          throw;
        }
        rh_graph* g = w->ctx->end_capture();
        w->step_graphs[key] = {g, op->grad_state()};
        w->ctx->launch(g);  // nothing ran while recording; step() already advanced the iteration counter
        w->graph_launches += 1;
        done = true;
      } else {
        if (w->seen_steps.size() >= kMaxSeenSteps) w->seen_steps.clear();
        w->seen_steps.insert(key);
      }
    }
    float loss;
    if (!done) {
      // launch by launch: the read-backs are started right behind the loss kernels and waited for after the backward
      // pass and the update are enqueued, so the host returns (and enqueues the next batch) while those still run
      op->forward(b, phase);
      op->loss_operator(0)->enqueue_output_categories(b);
      op->loss_operator(0)->enqueue_loss(b);
      op->loss_operator(0)->begin_fetch(b);
      op->backward(b);
      s->opt->step(op, fused != 0);
      loss = op->loss_operator(0)->finish_fetch(b);
    } else {
      op->loss_operator(0)->fetch_output_categories(b);
      loss = op->loss_operator(0)->fetch_loss();
    }
    const size_t correct = op->loss_operator(0)->accuracy_count(b);
    if (loss_out) *loss_out = loss;
    if (correct_out) *correct_out = (int32_t)correct;
  })
}


int rho_dataset_open(const char* source, const char* data_path, const char* labels_path, rho_dataset** out) {
  RHO_TRY({
    RHO_REQ(source && data_path && out);
    DataSourceConfig c;
    c.source = source;
    c.data_path = data_path;
    if (labels_path && *labels_path) { c.labels_path = labels_path; c.has_labels = true; }
    std::unique_ptr<rho_dataset> d(new rho_dataset());
    d->src = build_data_source(c);
    *out = d.release();
  })
}
int rho_dataset_open_from_file(const char* data_file_path, const char* key, rho_dataset** out) {
  RHO_TRY({
    RHO_REQ(data_file_path && key && out);
    std::unique_ptr<rho_dataset> d(new rho_dataset());
    d->src = build_data_source(DatasetConfig::open(data_file_path), key);
    *out = d.release();
  })
}
int rho_dataset_free(rho_dataset* d) { RHO_TRY({ delete d; }) }
int rho_dataset_num_samples(const rho_dataset* d, int64_t* out) { RHO_TRY({ RHO_REQ(d && out); *out = (int64_t)d->src->num_samples(); }) }
int rho_dataset_frame_dims(const rho_dataset* d, int32_t* w, int32_t* h, int32_t* c) {
  RHO_TRY({
    RHO_REQ(d && w && h && c);
    const Dims3 dims = d->src->frame_dims();
    *w = (int32_t)dims.w; *h = (int32_t)dims.h; *c = (int32_t)dims.c;
  })
}
int rho_dataset_get_sample(const rho_dataset* d, int64_t idx, uint8_t* frame_out, int32_t* category) {
  RHO_TRY({
    RHO_REQ(d && idx >= 0 && category);
    const uint8_t* f = nullptr;
    if (!d->src->get_sample((size_t)idx, &f, category)) panic("sample index out of range");
    if (frame_out) std::copy(f, f + d->src->frame_dims().len(), frame_out);
  })
}

int rho_sgd_train(rho_sgd* s, rho_worker* w, const rho_dataset* train, int train_order, uint64_t order_seed,
                  const rho_dataset* valid, const rho_train_config* cfg, rho_train_stats* stats_out) {
  RHO_TRY({
    RHO_REQ(s && w && train && cfg);
    RHO_REQ(train_order >= RHO_ORDER_SEQUENTIAL && train_order <= RHO_ORDER_CYCLIC_EPISODE);
    SgdTrainConfig c;
    c.init = cfg->resume_from >= 0 ? SgdTrainConfig::ResumeFrom : SgdTrainConfig::InitOrResume;
    c.resume_t = cfg->resume_from >= 0 ? (size_t)cfg->resume_from : 0;
    c.checkpoint_dir = cfg->checkpoint_dir ? cfg->checkpoint_dir : "";
    c.display_iters = (size_t)cfg->display_iters;
    c.checkpoint_iters = (size_t)cfg->checkpoint_iters;
    c.save_iters = (size_t)cfg->save_iters;
    c.valid_iters = (size_t)cfg->valid_iters;
    c.checkpoint_discard = cfg->checkpoint_discard != 0;
    c.max_iters = (size_t)cfg->max_iters;
    c.fused = cfg->fused != 0;
    const uint64_t seed[2] = {order_seed, order_seed ^ 0x9E3779B97F4A7C15ull};
    DataIter train_iter(train->src.get(), (DataIter::Kind)train_order, seed);
    std::unique_ptr<DataIter> valid_iter;
    if (valid) valid_iter.reset(new DataIter(valid->src.get(), DataIter::Sequential, seed));
    const SgdTrainStats st = sgd_train(*s->opt, *w->worker, train_iter, valid_iter.get(), c);
    if (stats_out) {
      stats_out->iters = (int64_t)st.iters;
      stats_out->epochs = (int64_t)st.epochs;
      stats_out->last_loss = st.last_loss;
      stats_out->last_error = st.last_error;
      stats_out->valid_runs = (int64_t)st.valid_runs;
      stats_out->valid_loss = st.valid_loss;
      stats_out->valid_error = st.valid_error;
      std::snprintf(stats_out->log_path, sizeof(stats_out->log_path), "%s", st.log_path.c_str());
    }
  })
}
int rho_sgd_validate(rho_worker* w, const rho_dataset* valid, float* loss, float* accuracy) {
  RHO_TRY({
    RHO_REQ(w && valid);
    const uint64_t seed[2] = {1, 2};
    DataIter it(valid->src.get(), DataIter::Sequential, seed);
    sgd_validate(*w->worker, it, loss, accuracy);
  })
}
}  // extern "C"
