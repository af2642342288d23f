// Host-side operator layer: a C++ mirror of the reference's Rust operator API for the
// single-GPU hot path, written only against the C ABI of include/rembrandt_hip.h.
//
// Mirrors (paths relative to the reference tree):
//   Operator / InputOperator traits ........ src/operator/mod.rs:61-109
//   OpCapability, OpPhase, Regularization,
//   ActivationFunction, ParamsInit ......... src/operator/mod.rs:233-297
//   Data3dOperator + preprocessing ......... src/operator/mod.rs:395-836
//   DropoutOperator ........................ src/operator/mod.rs:2134-2255
//   encode/decode_params/state ............. src/operator/mod.rs:1008-1073, 1594-1661
//   checkpoint / rollback files ............ src/worker/gossip_dist.rs:1230-1413
//   AffineOperator ......................... src/operator/mod.rs:843-1364
//   Conv2dOperator ......................... src/operator/mod.rs:1366-2003
//   Pool2dOperator ......................... src/operator/mod.rs:2005-2132
//   LossOperator, SoftmaxKLLossOperator .... src/operator/loss.rs:20-262
//   SequentialOperatorConfig / Worker ...... src/operator/worker.rs:133-477
//   gen-2 layer methods backward(batch, scale),
//   descend, reset_gradients; arch fan-out . src/layer_new.rs:537-617, 1044-1154; src/arch_new.rs:527-552
//   gen-2 minibatch update ................. src/opt_new.rs:304-325
//   SgdOptConfig, StepSizeSchedule,
//   Momentum, the update block ............. src/opt/sgd/mod.rs:20-147, src/opt/sgd/new.rs:345-495
//
// Error behaviour: like the reference, which panics on every native error and on every violated
// precondition, these classes throw std::runtime_error; nothing is recoverable.
// Ownership: each operator owns its out_act / out_delta / parameter / gradient / momentum
// buffers; neighbours share them by reference count (Rc<RefCell<DeviceBuffer>> in the reference).
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/rembrandt_hip.h"

namespace rembrandt {

[[noreturn]] void panic(const std::string& msg);
void unwrap(int code, const char* what);  // throws unless code == 0

// ---- device runtime (stands in for array_cuda::device::{context,memory}) --------------------
class DeviceContext {
 public:
  explicit DeviceContext(int device_idx);
  ~DeviceContext();
  DeviceContext(const DeviceContext&) = delete;
  DeviceContext& operator=(const DeviceContext&) = delete;
  rh_stream_t stream() const { return rh_ctx_stream(ctx_); }
  rh_stream_t aux_stream() const;  // second stream for launches that may overlap the main one
  void fork() const;               // aux waits for main
  void join() const;               // main waits for aux
  // Recording of the launches made on both streams into a replayable graph (rh_ctx_begin_capture / _end_capture).
  void begin_capture() const;
  rh_graph* end_capture() const;   // instantiated recording
  void abort_capture() const;      // discards the recording (after a failure inside it)
  void launch(rh_graph* g) const;
  rh_ctx* raw() const { return ctx_; }
  void sync() const;

 private:
  rh_ctx* ctx_;
};

// Page-locked host bytes (zero-filled): staging for per-batch copies to the device.
class PinnedBytes {
 public:
  PinnedBytes(size_t len, std::shared_ptr<DeviceContext> ctx);
  ~PinnedBytes();
  PinnedBytes(const PinnedBytes&) = delete;
  PinnedBytes& operator=(const PinnedBytes&) = delete;
  uint8_t* data() { return ptr_; }
  const uint8_t* data() const { return ptr_; }
  size_t size() const { return len_; }

 private:
  uint8_t* ptr_ = nullptr;
  size_t len_;
  std::shared_ptr<DeviceContext> ctx_;
};

template <class T>
class DeviceBuffer {
 public:
  // zero-filled, like DeviceBuffer::zeros(len, ctx)
  DeviceBuffer(size_t len, std::shared_ptr<DeviceContext> ctx) : len_(len), ctx_(std::move(ctx)) {
    void* p = nullptr;
    unwrap(rh_malloc(ctx_->raw(), len * sizeof(T), &p), "rh_malloc");
    ptr_ = static_cast<T*>(p);
  }
  ~DeviceBuffer() { rh_free(ctx_->raw(), ptr_); }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  T* as_mut_ptr() { return ptr_; }
  const T* as_ptr() const { return ptr_; }
  size_t len() const { return len_; }
  void sync_load(const T* host, size_t n) { unwrap(rh_load_sync(ctx_->raw(), ptr_, host, n * sizeof(T)), "sync_load"); }
  void sync_store(T* host, size_t n) const { unwrap(rh_store_sync(ctx_->raw(), host, ptr_, n * sizeof(T)), "sync_store"); }

 private:
  T* ptr_ = nullptr;
  size_t len_;
  std::shared_ptr<DeviceContext> ctx_;
};

typedef std::shared_ptr<DeviceBuffer<float>> SharedDeviceBuf;

// ---- small enums / value types ------------------------------------------------------------------
enum class OpCapability { Forward, Backward };
inline bool backward_enabled(OpCapability c) { return c != OpCapability::Forward; }

struct OpPhase {
  bool training;
  size_t t;
  static OpPhase Inference() { return {false, 0}; }
  static OpPhase Training(size_t t) { return {true, t}; }
};

struct Regularization {  // only L2 exists (src/operator/mod.rs:267-270)
  float l2_reg_coef;
  static Regularization L2(float c) { return {c}; }
};

enum class ActivationFunction { Identity, Rect, Logistic, Tanh };  // only Identity and Rect are implemented

struct ParamsInit {
  enum Kind { Disabled, Uniform, Normal, Xavier, KaimingFwd } kind;
  float value;  // half_range (Uniform) or std (Normal)
  static ParamsInit MakeDisabled() { return {Disabled, 0.0f}; }
  static ParamsInit MakeUniform(float half_range) { return {Uniform, half_range}; }
  static ParamsInit MakeNormal(float std) { return {Normal, std}; }
  static ParamsInit MakeXavier() { return {Xavier, 0.0f}; }
  static ParamsInit MakeKaimingFwd() { return {KaimingFwd, 0.0f}; }
};

enum class PoolOperation { Max, Average };

struct Dims3 {  // (width, height, channels), as in the reference
  size_t w, h, c;
  size_t len() const { return w * h * c; }
};

// ---- operator configs ---------------------------------------------------------------------------
// Data3dPreproc (src/operator/mod.rs:395-423).  AddPixelwiseColorNoise and NormalizePixelwise are
// `unimplemented!()` in the reference and are not offered here.
struct Data3dPreproc {
  enum Kind { Crop, FlipX, SubtractElemwiseMean, AddPixelwisePCALightingNoise } kind;
  size_t crop_width = 0, crop_height = 0;      // Crop
  std::string mean_path;                       // SubtractElemwiseMean: an NdArray file of in_dims ...
  std::vector<float> mean_values;              // ... or the values themselves (in_dims.len() floats, W fastest)
  float singular_vecs[3][3] = {{0}};           // AddPixelwisePCALightingNoise
  float singular_vals[3] = {0};
  float std_dev = 0.0f;
};

struct Data3dOperatorConfig {
  Dims3 in_dims;
  bool normalize;  // u8 frames are scaled by 1/255 when set (cast_bytes_normalized)
  std::vector<Data3dPreproc> preprocs;
  Dims3 get_out_dims() const;  // src/operator/mod.rs:432-462
};

struct AffineOperatorConfig {
  size_t in_channels, out_channels;
  ActivationFunction act_func;
  ParamsInit init_weights;
  size_t params_len() const { return in_channels * out_channels + out_channels; }
};

struct Conv2dOperatorConfig {
  Dims3 in_dims;
  size_t conv_size, conv_stride, conv_pad, out_channels;
  ActivationFunction act_func;
  ParamsInit init_weights;
  Dims3 get_out_dims() const;
  size_t params_len() const { return conv_size * conv_size * in_dims.c * out_channels + out_channels; }
};

struct Pool2dOperatorConfig {
  Dims3 in_dims;
  size_t pool_size, pool_stride, pool_pad;
  PoolOperation pool_op;
  ActivationFunction act_func;  // present in the reference's struct, never read there either
  bool ceil_mode;               // gen-1 extent (src/layer.rs:1741-1747); false = operator-style floor
  Dims3 get_out_dims() const;
};

struct DropoutOperatorConfig {  // src/operator/mod.rs:2134-2138
  size_t channels;
  float drop_ratio;
};

// The `local_res_norm` layer type of the `.model` grammar (examples/imagenet_alexnet.model:31-37); the
// reference's own layer for it is an empty stub (src/layer.rs:1846-1899).
struct LocalResNormOperatorConfig {
  Dims3 in_dims;
  size_t cross_size;
  float scale, power, min_div;
};

// How the moving batch-norm statistics weigh the newest batch at iteration t (src/operator/conv.rs:52-73).
struct BNormMovingAverage {
  enum Kind { Cumulative, Exponential } kind;
  double ema_factor;
  static BNormMovingAverage MakeCumulative() { return {Cumulative, 0.0}; }
  static BNormMovingAverage MakeExponential(double f) { return {Exponential, f}; }
  double at_iter(size_t t) const {
    if (kind == Cumulative) return 1.0 / (1.0 + (double)t);
    return t == 0 ? 1.0 : ema_factor;
  }
};

// conv (no bias) -> spatial batch norm -> activation (src/operator/conv.rs:75-104)
struct BNormConv2dOperatorConfig {
  Dims3 in_dims;
  size_t conv_size, conv_stride, conv_pad, out_channels;
  BNormMovingAverage bnorm_mov_avg;
  double bnorm_epsilon;
  ActivationFunction act_func;
  ParamsInit init_weights;
  Dims3 get_out_dims() const;
  size_t params_len() const { return conv_size * conv_size * in_dims.c * out_channels + 4 * out_channels; }
};

// y = act(x + BN2(conv3x3(act(BN1(conv3x3(x)))))), channels and extent unchanged (src/operator/conv.rs:914-935)
struct StackResConv2dOperatorConfig {
  Dims3 in_dims;
  BNormMovingAverage bnorm_mov_avg;
  double bnorm_epsilon;
  ActivationFunction act_func;
  ParamsInit init_weights;
  Dims3 get_out_dims() const { return in_dims; }
  size_t params_len() const { return 2 * (3 * 3 * in_dims.c * in_dims.c + 4 * in_dims.c); }
};

// y = act(BN3(conv1x1/s(x)) + BN2(conv3x3(act(BN1(conv3x3/s(x)))))); s = 1 when the extent is kept, 2 when it halves
// (src/operator/conv.rs:2184-2208, 2331-2338)
struct ProjStackResConv2dOperatorConfig {
  Dims3 in_dims, out_dims;
  BNormMovingAverage bnorm_mov_avg;
  double bnorm_epsilon;
  ActivationFunction act_func;
  ParamsInit init_weights;
  Dims3 get_out_dims() const { return out_dims; }
  size_t params_len() const {
    return 3 * 3 * in_dims.c * out_dims.c + 3 * 3 * out_dims.c * out_dims.c + in_dims.c * out_dims.c + 12 * out_dims.c;
  }
};

struct CategoricalLossConfig {
  size_t num_categories;
};

struct OperatorConfig {
  enum Kind { Data3d, Affine, Conv2d, Pool2d, SoftmaxKLLoss, Dropout, LocalResNorm, BNormConv2d, StackResConv2d,
              ProjStackResConv2d } kind;
  BNormConv2dOperatorConfig bnorm_conv2d;
  StackResConv2dOperatorConfig stack_res_conv2d;
  ProjStackResConv2dOperatorConfig proj_stack_res_conv2d;
  Data3dOperatorConfig data3d;
  AffineOperatorConfig affine;
  Conv2dOperatorConfig conv2d;
  Pool2dOperatorConfig pool2d;
  CategoricalLossConfig loss;
  DropoutOperatorConfig dropout;
  LocalResNormOperatorConfig lrn;
  size_t params_len() const;
};

// How kernels are scheduled inside the operators.  Both modes produce the same buffers at every
// point where the reference's operators expose them.
struct ExecOptions {
  // A whole train step (forward, loss kernels, backward, update) recorded once per (batch size, step scalars) and
  // replayed as one graph launch: for launch-bound networks.  Steps whose launch arguments change from one step to
  // the next (random preprocessing, dropout streams, a cumulative batch-norm average) run launch by launch.
  bool graph_steps = false;
  bool fuse_epilogue = true;  // conv bias + ReLU in the conv epilogue instead of K1 -> K2 -> K3
  bool bf16_forward = false;  // conv forward on bf16-rounded operands with fp32 accumulation (inference mode)
  // Set by the worker for forward-only chains with bf16_forward: neighbouring convolutions (and max-pools between
  // them) hand each other packed bf16 activations instead of fp32 ones (same values as rounding the fp32 ones).
  bool bf16_packed_chain = false;
  // Conv backward: filter and bias gradients on the context's second stream beside the data gradient on the
  // main one (the bandwidth-bound operand copies of one hide behind the other's contraction); joined at the end
  // of SequentialOperatorWorker::backward.
  bool overlap_backward = true;
  // A train step's classifier tail (two affine layers in front of the softmax loss, small enough for a sample's chain
  // to fit one block) as one launch for forward + loss + data gradients and one for the parameter gradients, instead
  // of ten launches of a few microseconds of work each; only inside armed train steps with fused epilogues.  Same
  // buffers with the same meaning at every point the operators expose; sums in a different (fixed) order.
  bool fuse_tail = true;
  // 3x3 stride-1 convolutions of 64 channels and more (all three passes) by Winograd F(2x2, 3x3), where the library
  // takes that form by itself; false keeps the direct form everywhere (RH_ALGO_DIRECT).
  bool winograd = true;
};

// ---- Operator trait -------------------------------------------------------------------------------
class Operator {
 public:
  virtual ~Operator() {}
  virtual size_t batch_size() const = 0;
  virtual SharedDeviceBuf get_output_vars() const { return nullptr; }
  virtual SharedDeviceBuf get_output_deltas() const { return nullptr; }
  virtual void init_params(const uint64_t /*shared_seed*/[2]) {}
  virtual void forward(size_t batch_size, OpPhase phase) = 0;
  virtual void backward(size_t batch_size) = 0;
  virtual void regularize(Regularization) {}
  virtual void accumulate_grads(float /*scale*/, float /*momentum*/) {}
  virtual void update_params(float /*scale*/) {}
  virtual void update_params2(float /*grad_scale*/, float /*update_scale*/) {}
  virtual void save_params() {}
  virtual void restore_params() {}
  virtual void reset() {}
  // The second-generation layer API (src/layer_new.rs:43-60), in which the gradient buffer doubles as the momentum
  // buffer.  backward_scaled: `scale` is the factor of the filter and bias gradients of a convolution
  // (layer_new.rs:1093-1108); an affine layer takes the argument and accumulates with factor 1, as the reference's
  // does (layer_new.rs:583-584); operators without parameters have nothing to scale.
  virtual void backward_scaled(size_t batch_size, float /*scale*/) { backward(batch_size); }
  // g += l2*W (if l2 > 0); W -= scale*g  (layer_new.rs:596-617, 1133-1154).  `fused`: one pass instead of two.
  virtual void descend(float /*scale*/, float /*l2_reg_coef*/, bool /*fused*/) {}
  // g *= scale: with scale = momentum the buffer carries the velocity into the next minibatch (layer_new.rs:589-594).
  virtual void reset_gradients(float /*scale*/) {}
  // Fused regularize -> accumulate_grads(scale, momentum) -> update_params(apply) -> reset in
  // one pass per tensor (same arithmetic, 24 instead of 52 bytes per parameter).
  virtual void fused_sgd_step(float /*l2*/, float /*scale*/, float /*momentum*/, float /*apply*/) {}
  // The {W, g, v} blocks that fused_sgd_step(l2, ...) would update, each with the l2 factor that applies to it, so that
  // a chain of operators can take the step in one launch per stream (rh_sgd_momentum_step_multi).
  virtual void sgd_tensors(float /*l2*/, std::vector<rh_sgd_tensor>& /*out*/) {}
  // True while the operator's gradient buffers stand for zeros without holding them (after a multi-tensor step that
  // did not zero them): its next backward pass overwrites instead of accumulating.  Part of what decides which
  // launches a step makes, hence of the key a recorded step is filed under.
  virtual bool grads_stale() const { return false; }
  // A recorded step was replayed: the host did not run the calls that flip this state, so it is set to what the
  // recording left behind.
  virtual void set_grads_stale(bool /*stale*/) {}
  // A consumer that can apply this operator's activation backward mask itself (max-pool backward folds the ReLU
  // mask) asks for it at construction; an operator that agrees skips its own mask pass in backward().  The
  // out_delta buffer holds the same values after the chain's backward either way.
  virtual bool fold_activation_backward() { return false; }
  // Packed bf16 activations (ExecOptions::bf16_packed_chain).  A convolution that reads a packed input asks the
  // operator below, at construction, whether it can write its output in that form (can_emit_packed) and, if so, for
  // the buffer (emit_packed, with the zero border the consumer's padding needs).  From then on the producer's forward
  // writes the packed buffer instead of its fp32 out_act; buffer(0) still answers with fp32 values (the bf16 values,
  // unpacked on demand).
  virtual bool can_emit_packed() const { return false; }
  virtual std::shared_ptr<DeviceBuffer<uint8_t>> emit_packed(int /*halo*/) { return nullptr; }
  // Switches the second-stream placement of gradient kernels on or off at run time (no effect on results, nor on
  // operators built without it).
  virtual void set_overlap_backward(bool /*on*/) {}
  // An operator whose fused SGD step may run on the context's second stream (large parameter blocks that the
  // next forward pass needs late: the affine layers) says so; the worker then joins the streams before that
  // operator's next forward and before anything else touches parameters.
  virtual bool updates_on_second_stream() const { return false; }
  // Whether forward / backward in this phase make the same launches with the same arguments every step, so that a
  // recording of one step can stand for the next.
  virtual bool graph_safe(OpPhase /*phase*/) const { return true; }
  // Parameter / optimizer-state blobs: a sequence of serialised NdArrays (weights then bias; for the state the
  // momentum buffers).  decode_* return the number of bytes consumed (src/operator/mod.rs:1008-1073).
  virtual void encode_params(std::vector<uint8_t>& /*blob*/) {}
  virtual size_t decode_params(const uint8_t* /*blob*/, size_t /*len*/) { return 0; }
  virtual void encode_state(std::vector<uint8_t>& /*blob*/) {}
  virtual size_t decode_state(const uint8_t* /*blob*/, size_t /*len*/) { return 0; }
  // Device views for inspection: 0 out_act, 1 out_delta, 2 weights, 3 bias, 4 grad_weights,
  // 5 grad_bias, 6 acc_grad_weights, 7 acc_grad_bias.  Returns false if the operator has no such buffer.
  // The batch-normalised operators number their conv + batch-norm units u = 0, 1, 2 and answer 100*u + id with
  // id = 2 weights, 4 grad_weights, 6 acc_grad_weights, 8 bn_scale, 9 bn_bias, 10 bn_scale_grad, 11 bn_bias_grad,
  // 12 bn_running_mean, 13 bn_running_ivar, 14 bn_cached_mean, 15 bn_cached_ivar, 16 acc_bn_scale_grad,
  // 17 acc_bn_bias_grad, 18 the unit's conv output (before the batch norm), 19 the gradient w.r.t. it; 30 / 31 are
  // the activation between the two stacked units and its gradient.
  virtual bool buffer(int which, float** ptr, size_t* len) {
    (void)which; (void)ptr; (void)len;
    return false;
  }
  virtual const char* kind() const = 0;
};

class InputOperator : public Operator {
 public:
  virtual uint8_t* expose_host_frame_buf(size_t batch_idx) = 0;
  virtual void load_frames(size_t batch_size) = 0;
  // Synthetic fp32 frames (N(0,1) inputs of the benchmark configs): bypasses the u8 cast.
  virtual void load_frames_f32(const float* host, size_t batch_size) = 0;
  virtual size_t in_frame_len() const = 0;  // bytes per staged frame
  // Which of the two loaders filled the frames that the next forward() reads (0: load_frames, u8 cast on the device;
  // 1: load_frames_f32): forward() makes different launches for the two, so a recorded step is valid for one only.
  virtual int input_mode() const = 0;
  // What the last forward() drew for its random preprocessing steps: crop offsets (of the last Crop), whether
  // the batch was flipped, and the 3*batch PCA lighting coefficients (empty if that step is absent or idle).
  virtual void last_preproc_draws(size_t* crop_off_w, size_t* crop_off_h, bool* flipped, std::vector<float>* alphas) const = 0;
  virtual Dims3 out_dims() const = 0;
};

class LossOperator : public Operator {
 public:
  virtual void stage_label(size_t batch_idx, int32_t category) = 0;
  virtual void load_labels(size_t batch_size) = 0;
  virtual void stage_weight(size_t batch_idx, float weight) = 0;
  virtual void load_weights(size_t batch_size) = 0;
  virtual float store_loss(size_t batch_size) = 0;
  // Second-generation loss bookkeeping (src/layer_new.rs:2103-2134): the loss is summed over batches on the device
  // until reset_loss; accumulate_loss adds this batch's sum_n -w_n log p[n, y_n]; store_accumulated_loss reads it.
  virtual void reset_loss(size_t batch_size) = 0;
  virtual void accumulate_loss(size_t batch_size) = 0;
  virtual float store_accumulated_loss() = 0;
  virtual void store_output_categories(size_t batch_size) = 0;
  // The two halves of store_loss / store_output_categories: enqueue_* launches the kernels that leave the result in
  // device buffers nothing else writes, fetch_* copies it to the host (blocking).  A caller may enqueue more work
  // (the backward pass) in between, so the GPU does not idle during the read-backs.
  virtual void enqueue_loss(size_t batch_size) = 0;
  virtual float fetch_loss() = 0;
  virtual void enqueue_output_categories(size_t batch_size) = 0;
  virtual void fetch_output_categories(size_t batch_size) = 0;
  // A third way to read both back: begin_fetch (after the two enqueue_* calls) starts their copies to page-locked
  // host memory on the context's copy stream, behind the kernels enqueued so far and beside whatever is enqueued
  // next; finish_fetch waits for the copies only, leaves the categories where get_output_categories finds them and
  // returns the loss.  The host then runs ahead of the GPU by the work enqueued in between.
  virtual void begin_fetch(size_t batch_size) = 0;
  virtual float finish_fetch(size_t batch_size) = 0;
  virtual const int32_t* get_output_categories(size_t batch_size) const = 0;
  virtual size_t accuracy_count(size_t batch_size) const = 0;
  // A train step asks the loss operator for its probabilities, predicted categories, loss and delta in a fixed
  // order with nothing in between that changes their inputs (labels and weights are loaded before the step).  While
  // armed, a training-phase forward() produces all four in one launch, and the enqueue_output_categories,
  // enqueue_loss and backward calls that follow it launch nothing.  Returns false where there is no such form.
  virtual bool arm_train_step(bool on) { (void)on; return false; }
};

// ---- graph ----------------------------------------------------------------------------------------
class SequentialOperatorConfig {
 public:
  OperatorConfig input_op;
  bool has_input = false;
  std::vector<OperatorConfig> hidden_ops;
  OperatorConfig loss_op;
  bool has_loss = false;

  size_t params_len() const;
  SequentialOperatorConfig& data3d(const Data3dOperatorConfig& cfg);
  SequentialOperatorConfig& affine(const AffineOperatorConfig& cfg);
  SequentialOperatorConfig& conv2d(const Conv2dOperatorConfig& cfg);
  SequentialOperatorConfig& pool2d(const Pool2dOperatorConfig& cfg);
  SequentialOperatorConfig& dropout(const DropoutOperatorConfig& cfg);              // src/operator/worker.rs:219-222
  SequentialOperatorConfig& local_res_norm(const LocalResNormOperatorConfig& cfg);
  SequentialOperatorConfig& bnorm_conv2d(const BNormConv2dOperatorConfig& cfg);                    // worker.rs:189-192
  SequentialOperatorConfig& stack_res_conv2d(const StackResConv2dOperatorConfig& cfg);            // worker.rs:194-197
  SequentialOperatorConfig& proj_stack_res_conv2d(const ProjStackResConv2dOperatorConfig& cfg);   // worker.rs:199-202
  SequentialOperatorConfig& softmax_kl_loss(const CategoricalLossConfig& cfg);
};

struct ClassifierTail;   // (operator.cpp)

class SequentialOperatorWorker : public Operator {
 public:
  SequentialOperatorWorker(const SequentialOperatorConfig& config, size_t batch_size, OpCapability capability,
                           const uint64_t shared_seed[2], std::shared_ptr<DeviceContext> context,
                           ExecOptions opts = ExecOptions());
  // OperatorWorker (src/operator/worker.rs:52-76); a single worker: rank 0 of 1.
  size_t num_workers() const { return 1; }
  size_t worker_rank() const { return 0; }
  const uint64_t* shared_seed() const { return shared_seed_; }
  InputOperator* input_operator() { return input_op_.get(); }
  size_t loss_count() const { return 1; }
  LossOperator* loss_operator(size_t rank);
  size_t hidden_count() const { return hidden_ops_.size(); }
  Operator* hidden_operator(size_t i) { return hidden_ops_.at(i).get(); }
  std::shared_ptr<DeviceContext> context() const { return context_; }

  size_t batch_size() const override { return batch_size_; }
  void init_params(const uint64_t shared_seed[2]) override;
  void forward(size_t batch_size, OpPhase phase) override;
  void backward(size_t batch_size) override;
  void regularize(Regularization reg) override;
  void accumulate_grads(float scale, float momentum) override;
  void update_params(float scale) override;
  void update_params2(float grad_scale, float update_scale) override;
  void save_params() override;
  void restore_params() override;
  void reset() override;
  // PipelineArchWorker::{backward, descend, reset_gradients} (src/arch_new.rs:534-551)
  void backward_scaled(size_t batch_size, float scale) override;
  void descend(float scale, float l2_reg_coef, bool fused) override;
  void reset_gradients(float momentum) override;
  void fused_sgd_step(float l2, float scale, float momentum, float apply) override;
  void set_overlap_backward(bool on) override;
  bool graph_safe(OpPhase phase) const override;
  // Operator::grads_stale of every hidden operator, and the way back.
  std::vector<char> grad_state() const;
  void set_grad_state(const std::vector<char>& state);
  // Joins the second stream if parameter updates are still in flight on it (called by every method but forward,
  // which joins lazily in front of the first operator concerned).
  void settle();
  // After a recording of a step was abandoned half-way: the launches that would have needed the join never ran.
  void forget_pending() { aux_pending_ = false; }
  // Arms (or disarms) the one-launch forms of a train step: the loss operator's, and the classifier tail's where the
  // chain ends in one (ExecOptions::fuse_tail).  While armed, forward() in the training phase also leaves the tail's
  // deltas behind and the following backward() of the same batch size only adds its parameter gradients.
  bool arm_train_step(bool on);
  bool has_fused_tail() const { return tail_ != nullptr; }
  const char* kind() const override { return "SequentialOperatorWorker"; }
  void encode_params(std::vector<uint8_t>& blob) override;
  size_t decode_params(const uint8_t* blob, size_t len) override;
  void encode_state(std::vector<uint8_t>& blob) override;
  size_t decode_state(const uint8_t* blob, size_t len) override;
  // Checkpoint files under `prefix` (src/worker/gossip_dist.rs:1230-1413): params.t_<t>.blob, the symlink
  // params.latest.blob, the text file `checkpoint` holding t (previous one kept as checkpoint.0), and
  // state.latest.blob.<rank> (params + momentum per operator).
  void checkpoint_params(size_t t, const std::string& prefix);
  void checkpoint_state(const std::string& prefix);
  bool can_rollback(const std::string& prefix, size_t* t) const;
  void rollback_params(const size_t* t /* nullptr = latest */, const std::string& prefix);
  void rollback_state(const std::string& prefix);
  // Uniform stream a DropoutOperator's last forward() consumed: (seed, stream id, first element).
  bool dropout_stream(size_t hidden_idx, uint64_t* seed, uint64_t* stream_id, uint64_t* first) const;

 private:
  size_t batch_size_;
  uint64_t shared_seed_[2];
  std::shared_ptr<DeviceContext> context_;
  std::unique_ptr<InputOperator> input_op_;
  std::vector<std::unique_ptr<Operator>> hidden_ops_;
  std::unique_ptr<LossOperator> loss_op_;
  bool aux_pending_ = false;
  std::shared_ptr<ClassifierTail> tail_;   // set when the chain ends in affine, affine, softmax loss of a fitting size
  bool tail_armed_ = false;
  size_t tail_done_ = 0;                   // batch size whose tail the last forward() ran in one launch; 0: none
};

// ---- SGD policy (src/opt/sgd/mod.rs:20-147) ---------------------------------------------------------
struct StepSizeSchedule {
  enum Kind { Constant, Anneal1, Anneal2, Anneal4, Decay, Inverse } kind;
  float step[5];     // step0..step4 (Constant: step[0]; Inverse: step[0] = init_step_size, step[1] = lambda)
  size_t iters[5];   // iters[i] = step{i}_iters for i = 1..4
  float at_iter(size_t t) const;
  static StepSizeSchedule MakeConstant(float s);
};

struct Momentum {
  enum Kind { Zero, Update, UpdateNesterov, Gradient, GradientNesterov } kind;
  float mu;
};

struct SgdOptConfig {
  size_t minibatch_size;
  StepSizeSchedule step_size;
  Momentum momentum;
  float l2_reg_coef;
};

// The per-minibatch update block of SgdOpt::train (src/opt/sgd/new.rs:345-495, 623-633) for one
// worker (no communication): regularize -> [Nesterov un-apply] -> iter_counter += 1 ->
// accumulate_grads -> update_params -> reset -> [Nesterov re-apply].
class SgdOpt {
 public:
  explicit SgdOpt(const SgdOptConfig& config) : config_(config) {}
  // Called once before the first minibatch (src/opt/sgd/new.rs:257-271).
  void begin(Operator* op);
  // `fused`: use Operator::fused_sgd_step where the flavour allows it (Zero, Update, Gradient).
  // `defer_reapply`: leave out the look-ahead `W += mu*v` that ends an UpdateNesterov step; the caller runs
  // reapply() after whatever must see the plain parameters (checkpoints, validation: new.rs:623-633).
  void step(Operator* op, bool fused, bool defer_reapply = false);
  void reapply(Operator* op);
  size_t iter_counter() const { return iter_counter_; }
  void set_iter_counter(size_t t) { iter_counter_ = t; }  // resuming from a checkpoint
  const SgdOptConfig& config() const { return config_; }

 private:
  SgdOptConfig config_;
  size_t iter_counter_ = 0;
};

// The per-minibatch block of the second-generation optimizer, SgdOptimization::train (src/opt_new.rs:304-325), for
// one worker: per batch forward -> backward(batch, 1.0) -> accumulate_loss with per-sample weights 1.0; at the end of
// a minibatch descend(step_size.at_iter(t) / minibatch_size, l2) -> reset_gradients(momentum) -> t += 1.
struct SgdOpt2Config {
  size_t minibatch_size;
  StepSizeSchedule step_size;
  float momentum;
  float l2_reg_coef;
};
class SgdOptimization {
 public:
  explicit SgdOptimization(const SgdOpt2Config& config) : config_(config) {}
  void begin(SequentialOperatorWorker* w);                       // reset_gradients(0), reset_loss (opt_new.rs:279-280)
  void batch(SequentialOperatorWorker* w, size_t batch_size);    // forward, backward(1.0), accumulate_loss
  void end_minibatch(SequentialOperatorWorker* w, bool fused);   // descend, reset_gradients, t += 1
  size_t iter_counter() const { return t_; }
  const SgdOpt2Config& config() const { return config_; }

 private:
  SgdOpt2Config config_;
  size_t t_ = 0;
};

// ---- NdArray (de)serialisation (header of tools/dump-array3d-header.rs:8-15) ------------------------------
// 'N' 'D' 0x00 0x01, u32 LE ndim, u64 LE dims[ndim], then the fp32 LE values in memory order (first index fastest).
void ndarray_serialize(std::vector<uint8_t>& out, const float* data, const size_t* dims, size_t ndim);
// Returns the bytes consumed; panics on a malformed header or a short blob.
size_t ndarray_deserialize(const uint8_t* blob, size_t len, std::vector<size_t>* dims, std::vector<float>* data);

}  // namespace rembrandt
