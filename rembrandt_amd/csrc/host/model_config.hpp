// Readers for the reference's two TOML config formats.
//   `.model`: [[layer]] tables -> layer list -> SequentialOperatorConfig   (src/config.rs:16-264)
//   `.data` : [dataset.<split>] tables -> source / paths                   (src/data_new.rs:297-342)
// The TOML subset the example files use is parsed by hand: comments, [table] and dotted
// [a.b] headers, [[array-of-tables]], key = value with strings, integers, floats, booleans,
// one-line arrays and one-line inline tables.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "operator.hpp"

namespace rembrandt {

struct TomlValue {
  enum Kind { None, String, Integer, Float, Boolean, Array, Table } kind = None;
  std::string s;
  long long i = 0;
  double f = 0.0;
  bool b = false;
  std::vector<TomlValue> array;
  std::vector<std::pair<std::string, TomlValue>> table;  // insertion order kept

  const TomlValue* lookup(const std::string& key) const;
  TomlValue* lookup_mut(const std::string& key);
  double as_float() const;  // accepts Float only, like toml::Value::as_float
};

TomlValue toml_parse(const std::string& text);  // throws std::runtime_error with a line number

struct LayerEntry {
  std::vector<std::string> names;
  std::vector<std::string> inputs;
  std::string type;  // data, fully_conn, conv2d, pool, local_res_norm, dropout, softmax_loss
  Dims3 in_dims;     // derived from the previous / named input layers
  Dims3 out_dims;
  // per-type fields (unused ones stay zero)
  size_t raw_width = 0, raw_height = 0, crop_width = 0, crop_height = 0, channels = 0;
  size_t out_channels = 0, conv_size = 0, conv_stride = 0, conv_pad = 0;
  size_t pool_size = 0, pool_stride = 0, pool_pad = 0, cross_size = 0, num_categories = 0;
  PoolOperation pool_kind = PoolOperation::Max;
  ActivationFunction act_func = ActivationFunction::Identity;
  ParamsInit init_weights = ParamsInit::MakeDisabled();
  float drop_ratio = 0.0f;
  float lrn_scale = 0.0f, lrn_power = 0.0f, lrn_min_div = 0.0f;
};

class ModelConfigFile {
 public:
  std::vector<LayerEntry> layers;
  static ModelConfigFile open(const std::string& path);
  static ModelConfigFile parse(const std::string& text);
  // Chain models only (one name per layer).  Pool layers keep the gen-1 ceil extent; a data layer whose crop
  // is smaller than its raw frame gets a Crop step; a fully_conn layer takes the flattened
  // width*height*channels of its input.
  SequentialOperatorConfig to_sequential_config() const;
};

struct DataSourceConfig {
  std::string source, data_path, labels_path, labels2_path;
  bool has_labels = false, has_labels2 = false;
};

class DatasetConfig {
 public:
  std::map<std::string, DataSourceConfig> datasets;
  static DatasetConfig open(const std::string& path);
  static DatasetConfig parse(const std::string& text);
};

}  // namespace rembrandt
