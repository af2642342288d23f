// Data sources, iterators and the training driver (see data_source.hpp).
#include "data_source.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstdio>
#include <cstring>

namespace rembrandt {

#define RB_ASSERT(cond) \
  do { if (!(cond)) ::rembrandt::panic(std::string("assertion failed: ") + #cond); } while (0)

MappedFile::MappedFile(const std::string& path, const char* what) {
  const int fd = ::open(path.c_str(), O_RDONLY);
  if (fd < 0) panic(std::string("failed to open ") + what + ": " + path);
  struct stat st;
  if (::fstat(fd, &st) != 0) { ::close(fd); panic(std::string("failed to stat ") + what + ": " + path); }
  size_ = (size_t)st.st_size;
  if (size_ > 0) {
    void* p = ::mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd, 0);
    if (p == MAP_FAILED) { ::close(fd); panic(std::string("failed to mmap buffer: ") + path); }
    data_ = static_cast<const uint8_t*>(p);
  }
  ::close(fd);
}

MappedFile::~MappedFile() {
  if (data_) ::munmap(const_cast<uint8_t*>(data_), size_);
}

namespace {
uint32_t be32(const uint8_t* p) { return (uint32_t)p[0] << 24 | (uint32_t)p[1] << 16 | (uint32_t)p[2] << 8 | (uint32_t)p[3]; }

// idx header (src/data_new.rs:680-745): u32 BE magic 0x0000 0x08 ndims, ndims u32 BE extents, then bytes.
struct IdxHeader { size_t n, frame_size, offset, ndims; size_t dims[4]; };
IdxHeader parse_idx(const MappedFile& f, const char* what) {
  if (f.size() < 4) panic(std::string(what) + ": truncated idx header");
  const uint32_t magic = be32(f.data());
  if (((magic >> 8) & 0xff) != 0x08) panic(std::string(what) + ": idx magic does not name unsigned bytes");
  IdxHeader h = IdxHeader();
  h.ndims = magic & 0xff;
  if (h.ndims != 1 && h.ndims != 3) panic(std::string(what) + ": unimplemented idx rank");
  if (f.size() < 4 * (1 + h.ndims)) panic(std::string(what) + ": truncated idx header");
  for (size_t d = 0; d < h.ndims; ++d) h.dims[d] = be32(f.data() + 4 * (1 + d));
  h.n = h.dims[0];
  h.frame_size = 1;
  for (size_t d = 1; d < h.ndims; ++d) h.frame_size *= h.dims[d];
  h.offset = 4 * (1 + h.ndims);
  if (f.size() - h.offset != h.n * h.frame_size) panic(std::string(what) + ": idx payload length does not match its header");
  return h;
}
}  // namespace

MnistDataSource::MnistDataSource(const DataSourceConfig& config) {
  data_file_.reset(new MappedFile(config.data_path, "mnist data file"));
  if (!config.has_labels) panic("mnist source needs a labels_path");
  labels_file_.reset(new MappedFile(config.labels_path, "mnist labels file"));
  const IdxHeader d = parse_idx(*data_file_, "mnist data file");
  if (d.ndims != 3) panic("mnist data file: expected a rank-3 idx file");
  const IdxHeader l = parse_idx(*labels_file_, "mnist labels file");
  if (l.ndims != 1) panic("mnist labels file: expected a rank-1 idx file");
  if (l.n != d.n) panic("mnist: data and labels disagree on the sample count");
  num_samples_ = d.n;
  frame_size_ = d.frame_size;
  data_off_ = d.offset;
  labels_off_ = l.offset;
  dims_ = {d.dims[2], d.dims[1], 1};  // (width, height, 1): dims[1] is rows
}

bool MnistDataSource::get_sample(size_t idx, const uint8_t** frame, int32_t* category) const {
  if (idx >= num_samples_) return false;
  *frame = data_file_->data() + data_off_ + idx * frame_size_;
  *category = (int32_t)labels_file_->data()[labels_off_ + idx];
  return true;
}

Cifar10DataSource::Cifar10DataSource(const DataSourceConfig& config) {
  file_.reset(new MappedFile(config.data_path, "cifar10 data file"));
  const size_t frame = 1 + 32 * 32 * 3;  // label byte, then 3 planes of 32x32 (src/data_new.rs:823-835)
  if (file_->size() % frame != 0) panic("cifar10 data file: length is not a multiple of 3073");
  num_samples_ = file_->size() / frame;
}

bool Cifar10DataSource::get_sample(size_t idx, const uint8_t** frame, int32_t* category) const {
  if (idx >= num_samples_) return false;
  const uint8_t* rec = file_->data() + idx * 3073;
  *category = (int32_t)rec[0];
  *frame = rec + 1;
  return true;
}

std::unique_ptr<DataSource> build_data_source(const DataSourceConfig& config) {
  if (config.source == "mnist") return std::unique_ptr<DataSource>(new MnistDataSource(config));
  if (config.source == "cifar10") return std::unique_ptr<DataSource>(new Cifar10DataSource(config));
  panic("unknown data source: '" + config.source + "'");
}

std::unique_ptr<DataSource> build_data_source(const DatasetConfig& datasets, const std::string& key) {
  auto it = datasets.datasets.find(key);
  if (it == datasets.datasets.end()) panic("dataset missing key: '" + key + "'");
  return build_data_source(it->second);
}

DataIter::DataIter(const DataSource* source, Kind kind, const uint64_t seed[2]) : source_(source), kind_(kind), s0_(seed[0]), s1_(seed[1]) {
  RB_ASSERT(source != nullptr);
  if (s0_ == 0 && s1_ == 0) s1_ = 0x9E3779B97F4A7C15ull;
}

uint64_t DataIter::next_u64() {  // xorshift128+
  uint64_t x = s0_;
  const uint64_t y = s1_;
  s0_ = y;
  x ^= x << 23;
  s1_ = x ^ y ^ (x >> 17) ^ (y >> 26);
  return s1_ + y;
}

void DataIter::reset() { drawn_ = 0; }

bool DataIter::next(const uint8_t** frame, int32_t* category) {
  const size_t n = source_->num_samples();
  if (n == 0 || drawn_ >= n) return false;
  size_t idx;
  switch (kind_) {
    case RandomEpisode: idx = (size_t)(next_u64() % (uint64_t)n); break;  // with replacement (src/data_new.rs:214-234)
    default: idx = drawn_; break;  // Sequential and CyclicEpisode visit 0..n-1; the caller's reset() makes the cycle
  }
  ++drawn_;
  last_idx_ = idx;
  return source_->get_sample(idx, frame, category);
}

// ---- training driver --------------------------------------------------------------------------------------
namespace {
double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
bool file_exists(const std::string& p) {
  struct stat st;
  return ::stat(p.c_str(), &st) == 0;
}
void mkdirs(const std::string& path) {
  std::string cur;
  for (size_t i = 0; i <= path.size(); ++i) {
    if ((i == path.size() || path[i] == '/') && !cur.empty()) ::mkdir(cur.c_str(), 0777);
    if (i < path.size()) cur.push_back(path[i]);
  }
}
void stage_sample(SequentialOperatorWorker& op, size_t batch_idx, const uint8_t* frame, int32_t category, float weight) {
  std::memcpy(op.input_operator()->expose_host_frame_buf(batch_idx), frame, op.input_operator()->in_frame_len());
  op.loss_operator(0)->stage_label(batch_idx, category);
  op.loss_operator(0)->stage_weight(batch_idx, weight);
}
}  // namespace

void sgd_validate(SequentialOperatorWorker& op, DataIter& valid, float* loss_out, float* accuracy_out) {
  const size_t batch_size = op.batch_size();
  const size_t num_shard = valid.num_shard_samples(), num_total = valid.num_total_samples();
  RB_ASSERT(num_total > 0);
  size_t acc_correct = 0, acc_total = 0, local_counter = 0, batch_counter = 0;
  float acc_loss = 0.0f;
  auto run = [&](size_t b) {
    op.input_operator()->load_frames(b);
    op.loss_operator(0)->load_labels(b);
    op.loss_operator(0)->load_weights(b);
    op.forward(b, OpPhase::Inference());
    op.loss_operator(0)->store_output_categories(b);
    acc_correct += op.loss_operator(0)->accuracy_count(b);
    acc_loss += op.loss_operator(0)->store_loss(b);
    acc_total += b;
  };
  valid.reset();
  const uint8_t* frame;
  int32_t category;
  RB_ASSERT(valid.frame_len() == op.input_operator()->in_frame_len());  // stage_shape (src/operator/mod.rs:826-830)
  while (local_counter < num_shard && valid.next(&frame, &category)) {
    stage_sample(op, batch_counter, frame, category, 1.0f / (float)num_total);
    ++local_counter;
    if (++batch_counter == batch_size) { run(batch_size); batch_counter = 0; }
  }
  if (batch_counter > 0) run(batch_counter);
  RB_ASSERT(local_counter == num_shard && acc_total == num_shard);
  if (loss_out) *loss_out = acc_loss;
  if (accuracy_out) *accuracy_out = (float)acc_correct / (float)acc_total;
}

SgdTrainStats sgd_train(SgdOpt& opt, SequentialOperatorWorker& op, DataIter& train, DataIter* valid, const SgdTrainConfig& cfg) {
  RB_ASSERT(cfg.max_iters > 0);
  const size_t batch_size = op.batch_size();
  const size_t minibatch_size = opt.config().minibatch_size;
  RB_ASSERT(minibatch_size % batch_size == 0);  // a minibatch is a whole number of forward/backward passes
  const float minibatch_weight = 1.0f / (float)minibatch_size;
  const size_t epoch_size = train.num_shard_samples();
  RB_ASSERT(epoch_size > 0);
  RB_ASSERT(train.frame_len() == op.input_operator()->in_frame_len());  // stage_shape (src/operator/mod.rs:826-830)
  SgdTrainStats stats;

  // trace log: first free name among trace_sgd.log, trace_sgd.log.1, ... (src/opt/sgd/new.rs:149-177)
  FILE* log = nullptr;
  if (!cfg.checkpoint_dir.empty()) {
    mkdirs(cfg.checkpoint_dir);
    for (int attempt = 0;; ++attempt) {
      stats.log_path = cfg.checkpoint_dir + "/trace_sgd.log" + (attempt ? "." + std::to_string(attempt) : "");
      if (!file_exists(stats.log_path)) break;
    }
    log = std::fopen(stats.log_path.c_str(), "w");
    if (!log) panic("SgdOpt: failed to open log file: " + stats.log_path);
    std::fprintf(log, "t,event,loss,error,elapsed\n");
    std::fflush(log);
  }
  struct Closer { FILE* f; ~Closer() { if (f) std::fclose(f); } } closer = {log};

  size_t init_t = 0;
  if (cfg.init == SgdTrainConfig::InitOrResume) {
    size_t t = 0;
    if (!cfg.checkpoint_dir.empty() && op.can_rollback(cfg.checkpoint_dir, &t)) {
      op.rollback_state(cfg.checkpoint_dir);
      init_t = t;
    } else {
      op.init_params(op.shared_seed());
    }
  } else {
    op.rollback_params(&cfg.resume_t, cfg.checkpoint_dir);
    init_t = cfg.resume_t;
  }
  opt.set_iter_counter(init_t);
  size_t elapsed_checkpoint_iters = init_t;
  opt.begin(&op);  // extra Nesterov momentum, reset()

  double minibatch_start = now_s();
  double minibatch_offset = 0.0;
  size_t mb_correct = 0, mb_total = 0, local_counter = 0, batch_counter = 0;
  float mb_loss = 0.0f;
  const uint8_t* frame;
  int32_t category;

  while (opt.iter_counter() < cfg.max_iters) {
    train.reset();
    while (opt.iter_counter() < cfg.max_iters && train.next(&frame, &category)) {
      stage_sample(op, batch_counter, frame, category, minibatch_weight);
      ++local_counter;
      stats.epochs = local_counter / epoch_size;
      ++batch_counter;
      if (batch_counter == batch_size) {
        op.input_operator()->load_frames(batch_size);
        op.loss_operator(0)->load_labels(batch_size);
        op.loss_operator(0)->load_weights(batch_size);
        op.forward(batch_size, OpPhase::Training(opt.iter_counter()));
        op.loss_operator(0)->store_output_categories(batch_size);
        mb_loss += op.loss_operator(0)->store_loss(batch_size);
        op.backward(batch_size);
        mb_correct += op.loss_operator(0)->accuracy_count(batch_size);
        mb_total += batch_size;
        batch_counter = 0;
      }
      if (local_counter % minibatch_size != 0) continue;

      opt.step(&op, cfg.fused, true);  // regularize, [Nesterov un-apply], iter += 1, accumulate, update, reset
      const size_t iter = opt.iter_counter();
      const double lap = now_s();
      stats.last_loss = mb_loss;
      stats.last_error = 1.0f - (float)mb_correct / (float)mb_total;
      if (log) {
        std::fprintf(log, "%zu,step,%.6f,%.4f,%.3f\n", iter, mb_loss, stats.last_error, lap - minibatch_start + minibatch_offset);
        if (cfg.display_iters && iter % cfg.display_iters == 0) std::fflush(log);
      }
      minibatch_start = now_s();
      minibatch_offset = 0.0;
      mb_correct = mb_total = 0;
      mb_loss = 0.0f;

      if (cfg.checkpoint_iters && iter % cfg.checkpoint_iters == 0) {  // one worker: the checkpoint is taken at once
        if (log) std::fflush(log);
        elapsed_checkpoint_iters += cfg.checkpoint_iters;
        if (cfg.checkpoint_discard) op.save_params();
        const double t0 = now_s();
        bool save_or_valid = false;
        if (cfg.save_iters && elapsed_checkpoint_iters % cfg.save_iters == 0) {
          save_or_valid = true;
          op.checkpoint_state(cfg.checkpoint_dir);
          op.checkpoint_params(elapsed_checkpoint_iters, cfg.checkpoint_dir);
        }
        if (valid && cfg.valid_iters && elapsed_checkpoint_iters % cfg.valid_iters == 0) {
          save_or_valid = true;
          const double v0 = now_s();
          float loss = 0.0f, acc = 0.0f;
          sgd_validate(op, *valid, &loss, &acc);
          stats.valid_runs += 1;
          stats.valid_loss = loss;
          stats.valid_error = 1.0f - acc;
          if (log) {
            std::fprintf(log, "%zu,valid,%.6f,%.4f,%.3f\n", iter, loss, 1.0f - acc, now_s() - v0);
            std::fflush(log);
          }
          batch_counter = 0;  // validation reused the staging buffers; a partial training batch cannot be pending here
        }
        if (cfg.checkpoint_discard) {
          op.restore_params();
          minibatch_start = now_s();
        } else if (save_or_valid) {
          minibatch_offset -= now_s() - t0;
        }
      }
      opt.reapply(&op);  // Nesterov look-ahead for the next iteration, after the checkpoint (new.rs:623-633)
    }
  }
  stats.iters = opt.iter_counter();
  return stats;
}

}  // namespace rembrandt
