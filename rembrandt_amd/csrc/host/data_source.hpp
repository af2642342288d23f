// Host-side data sources and sample iterators feeding the input operator: mirrors of the reference's
//   DataSource trait ............................ src/data_new.rs:414-423
//   MnistDataSource (idx files) ................. src/data_new.rs:648-795
//   Cifar10DataSource (binary batches) .......... src/data_new.rs:797-883
//   SampleIterator / RandomEpisodeIterator /
//   CyclicEpisodeIterator ....................... src/data_new.rs:124-280
//   DatasetConfig::build ........................ src/data_new.rs:343-357
// Every sample of these two sources is its own one-sample episode, so an "episode iterator" walks samples.
#pragma once
#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <vector>

#include "model_config.hpp"
#include "operator.hpp"

namespace rembrandt {

class DataSource {
 public:
  virtual ~DataSource() {}
  virtual size_t num_samples() const = 0;
  virtual Dims3 frame_dims() const = 0;  // (width, height, channels); bytes are W fastest, then H, then C
  // Pointer to the frame bytes (valid while the source lives) and the category; false past the end.
  virtual bool get_sample(size_t idx, const uint8_t** frame, int32_t* category) const = 0;
  virtual const char* kind() const = 0;
};

// A read-only memory map of a whole file.
class MappedFile {
 public:
  explicit MappedFile(const std::string& path, const char* what);
  ~MappedFile();
  MappedFile(const MappedFile&) = delete;
  MappedFile& operator=(const MappedFile&) = delete;
  const uint8_t* data() const { return data_; }
  size_t size() const { return size_; }

 private:
  const uint8_t* data_ = nullptr;
  size_t size_ = 0;
};

class MnistDataSource : public DataSource {
 public:
  explicit MnistDataSource(const DataSourceConfig& config);
  size_t num_samples() const override { return num_samples_; }
  Dims3 frame_dims() const override { return dims_; }
  bool get_sample(size_t idx, const uint8_t** frame, int32_t* category) const override;
  const char* kind() const override { return "mnist"; }

 private:
  std::unique_ptr<MappedFile> data_file_, labels_file_;
  size_t num_samples_ = 0, frame_size_ = 0, data_off_ = 0, labels_off_ = 0;
  Dims3 dims_ = {0, 0, 0};
};

class Cifar10DataSource : public DataSource {
 public:
  explicit Cifar10DataSource(const DataSourceConfig& config);
  size_t num_samples() const override { return num_samples_; }
  Dims3 frame_dims() const override { return {32, 32, 3}; }
  bool get_sample(size_t idx, const uint8_t** frame, int32_t* category) const override;
  const char* kind() const override { return "cifar10"; }

 private:
  std::unique_ptr<MappedFile> file_;
  size_t num_samples_ = 0;
};

// DatasetConfig::build: "mnist" | "cifar10" (the reference's "episodb" / "lmdb_caffe" stores are not part of this build).
std::unique_ptr<DataSource> build_data_source(const DataSourceConfig& config);
std::unique_ptr<DataSource> build_data_source(const DatasetConfig& datasets, const std::string& key);

// Sample order over one source.  reset() starts an epoch of num_samples() draws.
class DataIter {
 public:
  enum Kind { Sequential, RandomEpisode, CyclicEpisode };
  DataIter(const DataSource* source, Kind kind, const uint64_t seed[2]);
  size_t num_shard_samples() const { return source_->num_samples(); }
  size_t num_total_samples() const { return source_->num_samples(); }
  void reset();
  // Next sample of the epoch; false when the epoch is over.
  bool next(const uint8_t** frame, int32_t* category);
  size_t last_index() const { return last_idx_; }
  size_t frame_len() const { return source_->frame_dims().len(); }

 private:
  const DataSource* source_;
  Kind kind_;
  uint64_t s0_, s1_;
  size_t drawn_ = 0, last_idx_ = 0;
  uint64_t next_u64();
};

// ---- the SgdOpt::train / validate driver (src/opt/sgd/new.rs:209-766) for one worker ------------------------
struct SgdTrainConfig {
  enum Init { InitOrResume, ResumeFrom } init = InitOrResume;
  size_t resume_t = 0;
  std::string checkpoint_dir;
  size_t display_iters = 0;     // 0 = never
  size_t checkpoint_iters = 0;  // 0 = never: no save / validation points
  size_t save_iters = 0;
  size_t valid_iters = 0;
  bool checkpoint_discard = false;  // CheckpointBehavior::Discard: save_params before, restore_params after a checkpoint
  size_t max_iters = 0;             // the reference loops for ever; this driver stops after max_iters minibatches (total count)
  bool fused = true;                // fused SGD kernel where the momentum flavour allows it
};

struct SgdTrainStats {
  size_t iters = 0;          // iteration counter at return
  size_t epochs = 0;
  float last_loss = 0.0f;    // loss and error of the last minibatch
  float last_error = 0.0f;
  size_t valid_runs = 0;
  float valid_loss = 0.0f;   // of the last validation pass
  float valid_error = 0.0f;
  std::string log_path;
};

// Writes the CSV trace `t,event,loss,error,elapsed` (events "step" and "valid") to checkpoint_dir/trace_sgd.log
// (trace_sgd.log.N when that exists).
SgdTrainStats sgd_train(SgdOpt& opt, SequentialOperatorWorker& op, DataIter& train, DataIter* valid, const SgdTrainConfig& cfg);
void sgd_validate(SequentialOperatorWorker& op, DataIter& valid, float* loss, float* accuracy);

}  // namespace rembrandt
