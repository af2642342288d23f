/*
 * rembrandt_operator.h -- C ABI of the operator / graph / optimizer layer of librembrandt_hip.so.
 *
 * This is what a binding of the reference's *upper* boundary talks to: the Rust operator API
 * (Operator / InputOperator / LossOperator traits, src/operator/mod.rs:61-109 and
 * src/operator/loss.rs:20-39), the SequentialOperatorConfig builder and
 * SequentialOperatorWorker (src/operator/worker.rs:133-477) and the SGD policy
 * (src/opt/sgd/mod.rs:20-147, src/opt/sgd/new.rs:345-495).  Each function names the reference
 * method it stands for.  Dimension triples are (width, height, channels) as in the reference.
 *
 * Every function returns 0 on success.  The reference panics on errors; here a failed
 * precondition or native error returns RHO_E_PANIC and the text of the panic can be read with
 * rho_last_message() (per thread).
 */
#ifndef REMBRANDT_OPERATOR_H
#define REMBRANDT_OPERATOR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RHO_E_PANIC (-100)

typedef struct rho_config rho_config; /* SequentialOperatorConfig */
typedef struct rho_worker rho_worker; /* SequentialOperatorWorker + its DeviceContext */
typedef struct rho_sgd rho_sgd;       /* SgdOpt (update block only) */

const char* rho_last_message(void);

/* enums: ActivationFunction (mod.rs:282-288), ParamsInit (mod.rs:290-297), PoolOperation (mod.rs:2005-2009),
 * OpCapability (mod.rs:233-259), Momentum (opt/sgd/mod.rs:140-147), StepSizeSchedule (opt/sgd/mod.rs:44-80) */
enum { RHO_ACT_IDENTITY = 0, RHO_ACT_RECT = 1, RHO_ACT_LOGISTIC = 2, RHO_ACT_TANH = 3 };
enum { RHO_INIT_DISABLED = 0, RHO_INIT_UNIFORM = 1, RHO_INIT_NORMAL = 2, RHO_INIT_XAVIER = 3, RHO_INIT_KAIMING_FWD = 4 };
enum { RHO_POOL_MAX = 0, RHO_POOL_AVERAGE = 1 };
enum { RHO_CAP_FORWARD = 0, RHO_CAP_BACKWARD = 1 };
enum { RHO_MOM_ZERO = 0, RHO_MOM_UPDATE = 1, RHO_MOM_UPDATE_NESTEROV = 2, RHO_MOM_GRADIENT = 3, RHO_MOM_GRADIENT_NESTEROV = 4 };
enum { RHO_STEP_CONSTANT = 0, RHO_STEP_ANNEAL1 = 1, RHO_STEP_ANNEAL2 = 2, RHO_STEP_ANNEAL4 = 3, RHO_STEP_DECAY = 4, RHO_STEP_INVERSE = 5 };
/* buffers of an operator, for rho_worker_buffer */
enum { RHO_BUF_OUT_ACT = 0, RHO_BUF_OUT_DELTA = 1, RHO_BUF_WEIGHTS = 2, RHO_BUF_BIAS = 3, RHO_BUF_GRAD_WEIGHTS = 4,
       RHO_BUF_GRAD_BIAS = 5, RHO_BUF_ACC_GRAD_WEIGHTS = 6, RHO_BUF_ACC_GRAD_BIAS = 7,
       /* batch-normalised operators: RHO_BUF_UNIT*u + id addresses conv + batch-norm unit u = 0, 1, 2 (ids 2, 4, 6 as above) */
       RHO_BUF_BN_SCALE = 8, RHO_BUF_BN_BIAS = 9, RHO_BUF_BN_SCALE_GRAD = 10, RHO_BUF_BN_BIAS_GRAD = 11,
       RHO_BUF_BN_RUNNING_MEAN = 12, RHO_BUF_BN_RUNNING_IVAR = 13, RHO_BUF_BN_CACHED_MEAN = 14, RHO_BUF_BN_CACHED_IVAR = 15,
       RHO_BUF_ACC_BN_SCALE_GRAD = 16, RHO_BUF_ACC_BN_BIAS_GRAD = 17, RHO_BUF_PRE_ACT = 18, RHO_BUF_PRE_DELTA = 19,
       RHO_BUF_MID_ACT = 30, RHO_BUF_MID_DELTA = 31, RHO_BUF_UNIT = 100 };

/* ---- SequentialOperatorConfig builder (worker.rs:133-228) ---- */
int rho_config_new(rho_config** out);                                       /* ::new()            */
int rho_config_free(rho_config* cfg);
int rho_config_data3d(rho_config* cfg, int32_t w, int32_t h, int32_t c, int normalize);                /* .data3d()  */
int rho_config_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t conv_size,
                      int32_t conv_stride, int32_t conv_pad, int32_t out_channels, int act_func, int init_kind,
                      float init_value);                                                              /* .conv2d()  */
/* The batch-normalised operators of src/operator/conv.rs.  `mov_avg_kind`: RHO_BNORM_CUMULATIVE (newest batch weighs
 * 1/(1+t)) or RHO_BNORM_EXPONENTIAL (1 at t = 0, `ema_factor` afterwards), BNormMovingAverage::at_iter (:58-72). */
enum { RHO_BNORM_CUMULATIVE = 0, RHO_BNORM_EXPONENTIAL = 1 };
int rho_config_bnorm_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t conv_size,
                            int32_t conv_stride, int32_t conv_pad, int32_t out_channels, int mov_avg_kind,
                            double ema_factor, double epsilon, int act_func, int init_kind,
                            float init_value);                                            /* .bnorm_conv2d() (worker.rs:189)          */
int rho_config_stack_res_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int mov_avg_kind,
                                double ema_factor, double epsilon, int act_func, int init_kind,
                                float init_value);                                        /* .stack_res_conv2d() (worker.rs:194)      */
int rho_config_proj_stack_res_conv2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t out_w,
                                     int32_t out_h, int32_t out_c, int mov_avg_kind, double ema_factor, double epsilon,
                                     int act_func, int init_kind, float init_value);      /* .proj_stack_res_conv2d() (worker.rs:199) */
int rho_config_affine(rho_config* cfg, int32_t in_channels, int32_t out_channels, int act_func, int init_kind,
                      float init_value);                                                              /* .affine()  */
int rho_config_pool2d(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t pool_size,
                      int32_t pool_stride, int32_t pool_pad, int pool_op, int ceil_mode);              /* .pool2d()  */
int rho_config_softmax_kl_loss(rho_config* cfg, int32_t num_categories);
/* Data3dPreproc steps appended to the input operator's list, in call order (src/operator/mod.rs:395-423, 545-597).
 * Crop and FlipX draw once per forward() for the whole batch in Training and are centre / off in Inference;
 * SubtractElemwiseMean takes in_dims.len() values (W fastest) or an NdArray file; the mean is scaled by 1/255 when
 * the input operator normalises.  PCA lighting noise: 3x3 singular vectors (row j = vector j), 3 singular values. */
int rho_config_data3d_crop(rho_config* cfg, int32_t crop_width, int32_t crop_height);
int rho_config_data3d_flip_x(rho_config* cfg);
int rho_config_data3d_subtract_mean(rho_config* cfg, const float* mean, int64_t len);
int rho_config_data3d_subtract_mean_file(rho_config* cfg, const char* mean_path);
int rho_config_data3d_pca_lighting_noise(rho_config* cfg, const float* singular_vecs9, const float* singular_vals3,
                                         float std_dev);
int rho_config_dropout(rho_config* cfg, int32_t channels, float drop_ratio);                           /* .dropout() worker.rs:219 */
/* `local_res_norm` layers of the .model grammar (cross-channel; the reference's layer is a stub, layer.rs:1846-1899). */
int rho_config_local_res_norm(rho_config* cfg, int32_t in_w, int32_t in_h, int32_t in_c, int32_t cross_size, float scale,
                              float power, float min_div);                              /* .softmax_kl_loss() */
int rho_config_params_len(const rho_config* cfg, int64_t* out);                                       /* .params_len() */
/* Parses a `.model` file of the reference's grammar (src/config.rs:16-264) into a config.
 * batch-independent; returns the input dims through the config's data3d entry. */
int rho_config_from_model_file(const char* path, rho_config** out);

/* ---- SequentialOperatorWorker (worker.rs:230-477) ---- */
/* into_worker(): builds the chain on `device`.  exec_flags is a bit set (0 = the reference's kernel sequence in fp32):
 *   RHO_EXEC_FUSE_EPILOGUE  fold bias+ReLU into the conv epilogue (same buffers at every point the operators expose);
 *   RHO_EXEC_BF16_FORWARD   conv forward multiplies operands rounded to bf16 and accumulates in fp32
 *                           (forward-only inference mode; backward passes stay fp32 and read the same buffers);
 *   RHO_EXEC_OVERLAP_BACKWARD  conv filter / bias gradients run on a second stream beside the data gradient; the
 *                           streams are joined at the end of backward (same results: no kernel changes). */
#define RHO_EXEC_FUSE_EPILOGUE 0x1
#define RHO_EXEC_BF16_FORWARD  0x2
#define RHO_EXEC_OVERLAP_BACKWARD 0x4
/*   RHO_EXEC_GRAPH_STEPS    rho_sgd_train_batch records a whole step (forward, loss kernels, backward, update) into a HIP
 *                           graph the second time it sees a (batch size, optimizer scalars) combination and replays it
 *                           from then on: one launch per step instead of ~60 for a LeNet-sized network.  Steps whose
 *                           launch arguments change every step (random input preprocessing, dropout, a cumulative
 *                           batch-norm average, a step-size schedule at a boundary) run launch by launch as usual;
 *                           results are bit-identical either way. */
#define RHO_EXEC_GRAPH_STEPS 0x8
/*   RHO_EXEC_SEPARATE_TAIL  with RHO_EXEC_FUSE_EPILOGUE, rho_sgd_train_batch runs a classifier tail (affine -> affine ->
 *                           softmax loss, of at most 4096 x 2048 x 64 units and 2^17 first-layer weights) as two launches:
 *                           both layers' forward, the loss step and the data gradients per sample in one, the four
 *                           parameter gradients in another (rh_affine2_softmax_kl_step, rh_affine2_bwd_params), ten
 *                           launches otherwise.  Same buffers with the same meaning; sums in another order, so results
 *                           agree with the separate operators to rounding.  This flag keeps the separate operators. */
#define RHO_EXEC_SEPARATE_TAIL 0x10
/*   RHO_EXEC_DIRECT_CONV    3x3 and 5x5 stride-1 convolutions keep the direct form in all three passes (RH_ALGO_DIRECT).
 *                           Without it the library takes Winograd's F(2x2, 3x3) for 3x3 layers of 64 channels and more
 *                           (2.25x fewer multiply-adds) and for the forward pass of such 5x5 layers (1.56x fewer):
 *                           sums in another order, same tolerance against the oracle. */
#define RHO_EXEC_DIRECT_CONV 0x20
int rho_worker_new(const rho_config* cfg, int32_t batch_size, int capability, uint64_t seed0, uint64_t seed1,
                   int device, int exec_flags, rho_worker** out);
int rho_worker_free(rho_worker* w);
/* Number of rho_sgd_train_batch calls on this worker that ran as one graph launch (RHO_EXEC_GRAPH_STEPS). */
int rho_worker_graph_launches(rho_worker* w, int64_t* out);
/* Run-time switch of RHO_EXEC_OVERLAP_BACKWARD for a worker built with it (per-kernel timings are only meaningful
 * with it off: kernels that share the GPU stretch each other's durations). */
int rho_worker_set_overlap_backward(rho_worker* w, int on);
/* Output frame shape of the input operator (after crops), and what its last forward() drew. */
int rho_worker_input_out_dims(rho_worker* w, int32_t* out_w, int32_t* out_h, int32_t* out_c);
int rho_worker_last_preproc_draws(rho_worker* w, int32_t* crop_off_w, int32_t* crop_off_h, int* flipped, float* alphas,
                                  int64_t alphas_cap, int64_t* alphas_len);
/* The uniform stream a DropoutOperator's last Training forward() consumed: rand[i] = element (first + i) of
 * rh_rng_fill_uniform(seed, stream_id, ., ., 0, 1). */
int rho_worker_dropout_stream(rho_worker* w, int32_t hidden_idx, uint64_t* seed, uint64_t* stream_id, uint64_t* first);
/* encode/decode_params, encode/decode_state over all hidden operators (mod.rs:1008-1073, 1594-1661): a sequence of
 * NdArray records ('N','D',0,1, u32 rank, u64 dims, fp32 LE data).  Call encode with buf == NULL to get the size. */
int rho_worker_encode_params(rho_worker* w, uint8_t* buf, size_t cap, size_t* needed);
int rho_worker_decode_params(rho_worker* w, const uint8_t* blob, size_t len, size_t* consumed);
int rho_worker_encode_state(rho_worker* w, uint8_t* buf, size_t cap, size_t* needed);
int rho_worker_decode_state(rho_worker* w, const uint8_t* blob, size_t len, size_t* consumed);
/* Checkpoint files under `prefix` (worker/gossip_dist.rs:1230-1413): params.t_<t>.blob, params.latest.blob -> it,
 * `checkpoint` (text: t), checkpoint.0 (previous), state.latest.blob.<rank>. */
int rho_worker_checkpoint_params(rho_worker* w, int64_t t, const char* prefix);
int rho_worker_checkpoint_state(rho_worker* w, const char* prefix);
int rho_worker_can_rollback(rho_worker* w, const char* prefix, int64_t* t_or_minus1);
int rho_worker_rollback_params(rho_worker* w, int64_t t_or_minus1 /* -1 = latest */, const char* prefix);
int rho_worker_rollback_state(rho_worker* w, const char* prefix);
int rho_worker_hidden_count(rho_worker* w, int32_t* out);
int rho_worker_op_kind(rho_worker* w, int32_t hidden_idx, const char** out);
void* rho_worker_stream(rho_worker* w);                                      /* ctx.stream.ptr */
int rho_worker_sync(rho_worker* w);                                          /* ctx.sync()     */
int rho_worker_init_params(rho_worker* w, uint64_t seed0, uint64_t seed1);   /* Operator::init_params */
/* InputOperator (mod.rs:101-109) */
int rho_worker_expose_host_frame_buf(rho_worker* w, int32_t batch_idx, uint8_t** out);
int rho_worker_load_frames(rho_worker* w, int32_t batch_size);
int rho_worker_load_frames_f32(rho_worker* w, const float* host, int32_t batch_size);
/* LossOperator (loss.rs:20-39) */
int rho_worker_stage_label(rho_worker* w, int32_t batch_idx, int32_t category);
int rho_worker_load_labels(rho_worker* w, int32_t batch_size);
int rho_worker_stage_weight(rho_worker* w, int32_t batch_idx, float weight);
int rho_worker_load_weights(rho_worker* w, int32_t batch_size);
int rho_worker_store_loss(rho_worker* w, int32_t batch_size, float* out);
int rho_worker_store_output_categories(rho_worker* w, int32_t batch_size);
int rho_worker_get_output_categories(rho_worker* w, int32_t batch_size, int32_t* host_out);
int rho_worker_accuracy_count(rho_worker* w, int32_t batch_size, int32_t* out);
/* Operator (mod.rs:61-99), fanned out over the chain as in worker.rs:356-477 */
int rho_worker_forward(rho_worker* w, int32_t batch_size, int training, int64_t t);
int rho_worker_backward(rho_worker* w, int32_t batch_size);
int rho_worker_regularize(rho_worker* w, float l2_reg_coef);
int rho_worker_accumulate_grads(rho_worker* w, float scale, float momentum);
int rho_worker_update_params(rho_worker* w, float scale);
int rho_worker_update_params2(rho_worker* w, float grad_scale, float update_scale);
int rho_worker_save_params(rho_worker* w);
int rho_worker_restore_params(rho_worker* w);
int rho_worker_reset(rho_worker* w);
/* The second-generation layer / arch API over the same chain (src/layer_new.rs:43-60, src/arch_new.rs:527-552), where
 * the gradient buffers double as the momentum buffers:
 *   rho_worker_backward_scaled  PipelineArchWorker::backward(batch, scale): `scale` multiplies the filter and bias
 *                               gradients a convolution accumulates (layer_new.rs:1093-1108); affine layers accumulate
 *                               with factor 1 whatever it is (layer_new.rs:583-584); the loss layer ignores it (:1933)
 *   rho_worker_descend          g += l2*W (weights and bias, if l2 > 0); W -= scale*g   (layer_new.rs:596-617,1133-1154)
 *                               fused != 0: one pass per tensor instead of the BLAS-1 pair
 *   rho_worker_reset_gradients  g *= momentum                                            (layer_new.rs:589-594)
 *   rho_worker_reset_loss / _accumulate_loss / _store_accumulated_loss
 *                               the loss summed over batches on the device (layer_new.rs:2103-2134)
 * Batch-normalised operators have no second-generation counterpart and panic in descend / reset_gradients. */
int rho_worker_backward_scaled(rho_worker* w, int32_t batch_size, float scale);
int rho_worker_descend(rho_worker* w, float scale, float l2_reg_coef, int fused);
int rho_worker_reset_gradients(rho_worker* w, float momentum);
int rho_worker_reset_loss(rho_worker* w, int32_t batch_size);
int rho_worker_accumulate_loss(rho_worker* w, int32_t batch_size);
int rho_worker_store_accumulated_loss(rho_worker* w, float* out);
/* Device view of one buffer of hidden operator `hidden_idx` (-1: input operator's out_act,
 * hidden_count: the loss operator's probabilities).  Returns RHO_E_PANIC if there is no such buffer.
 * How long a pointer stays meaningful: the fused train step (rho_sgd_train_batch / rho_sgd_step with fused != 0) does
 * not write the zeros that the reference's `reset` leaves in grad_weights / grad_bias (which = 4, 5); it remembers that
 * they stand for zeros and its next backward pass overwrites them.  This call (and every other operator method that
 * looks at the gradients) makes the zeros real first, so what it shows is the reference's state; a gradient pointer kept
 * across a later fused step shows that step's gradients instead of zeros.  Ask again after each step, or use
 * rho_worker_read_buffer.  Likewise a weights / bias pointer (which = 2, 3) may be written through until the next
 * forward pass; a forward-only bf16 worker converts its filters when this call hands the pointer out, so write before
 * the next forward pass, not during it.  In a forward-only bf16 worker out_act (which = 0) of the operators between
 * convolutions holds the bf16 activations' values, unpacked when this call is made. */
int rho_worker_buffer(rho_worker* w, int32_t hidden_idx, int which, float** dptr, int64_t* len);
/* Blocking copies between host memory and such a buffer (sync_store / sync_load). */
int rho_worker_read_buffer(rho_worker* w, int32_t hidden_idx, int which, float* host, int64_t len);
int rho_worker_write_buffer(rho_worker* w, int32_t hidden_idx, int which, const float* host, int64_t len);

/* ---- SgdOpt update block (opt/sgd/new.rs:345-495, 623-633) ---- */
int rho_sgd_new(int32_t minibatch_size, int step_kind, const float* steps, const int64_t* step_iters, int momentum_kind,
                float mu, float l2_reg_coef, rho_sgd** out);
int rho_sgd_free(rho_sgd* s);
int rho_sgd_begin(rho_sgd* s, rho_worker* w);
int rho_sgd_step(rho_sgd* s, rho_worker* w, int fused);
int rho_sgd_iter_counter(rho_sgd* s, int64_t* out);
int rho_sgd_set_iter_counter(rho_sgd* s, int64_t t);   /* resuming: init_t of new.rs:231-252 */
int rho_sgd_step_size_at(rho_sgd* s, int64_t t, float* out);                 /* StepSizeSchedule::at_iter */
/* One whole training step on a staged batch, in the order of SgdOpt::train (new.rs:325-343 + the
 * update block): forward, store_output_categories, store_loss, backward, accuracy_count, step. */
int rho_sgd_train_batch(rho_sgd* s, rho_worker* w, int32_t batch_size, int fused, float* loss_out, int32_t* correct_out);

/* ---- SgdOptimization::train, the second-generation minibatch block (src/opt_new.rs:279-325) ----
 * rho_sgd2_begin: reset_gradients(0), reset_loss.  rho_sgd2_batch: forward(Training) -> backward(batch, 1.0) ->
 * accumulate_loss on a staged batch (per-sample weights 1.0, staged by the caller).  rho_sgd2_end_minibatch:
 * descend(step_size.at_iter(t) / minibatch_size, l2) -> reset_gradients(momentum) -> t += 1. */
typedef struct rho_sgd2 rho_sgd2;
int rho_sgd2_new(int32_t minibatch_size, int step_kind, const float* steps, const int64_t* step_iters, float momentum,
                 float l2_reg_coef, rho_sgd2** out);
int rho_sgd2_free(rho_sgd2* s);
int rho_sgd2_begin(rho_sgd2* s, rho_worker* w);
int rho_sgd2_batch(rho_sgd2* s, rho_worker* w, int32_t batch_size);
int rho_sgd2_end_minibatch(rho_sgd2* s, rho_worker* w, int fused);
int rho_sgd2_iter_counter(rho_sgd2* s, int64_t* out);

/* ---- data sources (src/data_new.rs:282-357, 648-883) ----
 * source: "mnist" (idx3-ubyte frames + idx1-ubyte labels) or "cifar10" (3073-byte records: label, 3 planes of 32x32).
 * rho_dataset_open_from_file reads a `.data` file ([dataset.<key>] source / data_path / labels_path). */
typedef struct rho_dataset rho_dataset;
int rho_dataset_open(const char* source, const char* data_path, const char* labels_path, rho_dataset** out);
int rho_dataset_open_from_file(const char* data_file_path, const char* key, rho_dataset** out);
int rho_dataset_free(rho_dataset* d);
int rho_dataset_num_samples(const rho_dataset* d, int64_t* out);
int rho_dataset_frame_dims(const rho_dataset* d, int32_t* w, int32_t* h, int32_t* c);
int rho_dataset_get_sample(const rho_dataset* d, int64_t idx, uint8_t* frame_out /* may be NULL */, int32_t* category);

/* ---- SgdOpt::train / validate for one worker (src/opt/sgd/new.rs:209-766) ----
 * Samples are staged through expose_host_frame_buf / stage_label / stage_weight(1/minibatch); every full batch runs
 * forward(Training{t}) -> arg-max, loss read-backs -> backward; every minibatch_size samples the update block runs
 * (gradients of the batches in between accumulate).  At every checkpoint_iters-th iteration: save_params (Discard),
 * checkpoint_state + checkpoint_params every save_iters, validation (Inference phase, weights 1/num_samples) every
 * valid_iters, restore_params (Discard).  The trace `t,event,loss,error,elapsed` goes to
 * <checkpoint_dir>/trace_sgd.log[.N].  init: resume_from < 0 = InitOrResume (rollback_state if a `checkpoint` file
 * exists, else init_params(shared_seed)), otherwise ResumeFrom{t}.  The reference loops for ever; max_iters ends it. */
#define RHO_ORDER_SEQUENTIAL     0  /* SampleIterator          */
#define RHO_ORDER_RANDOM_EPISODE 1  /* RandomEpisodeIterator: uniform with replacement */
#define RHO_ORDER_CYCLIC_EPISODE 2  /* CyclicEpisodeIterator   */
typedef struct rho_train_config {
  const char* checkpoint_dir;  /* NULL or "": no log, no checkpoints */
  int64_t resume_from;
  int64_t display_iters, checkpoint_iters, save_iters, valid_iters;
  int checkpoint_discard;
  int64_t max_iters;
  int fused;
} rho_train_config;
typedef struct rho_train_stats {
  int64_t iters, epochs;
  float last_loss, last_error;
  int64_t valid_runs;
  float valid_loss, valid_error;
  char log_path[512];
} rho_train_stats;
int rho_sgd_train(rho_sgd* s, rho_worker* w, const rho_dataset* train, int train_order, uint64_t order_seed,
                  const rho_dataset* valid /* may be NULL */, const rho_train_config* cfg, rho_train_stats* stats_out);
int rho_sgd_validate(rho_worker* w, const rho_dataset* valid, float* loss, float* accuracy);

#ifdef __cplusplus
}
#endif
#endif /* REMBRANDT_OPERATOR_H */
