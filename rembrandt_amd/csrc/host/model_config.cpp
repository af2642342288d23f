#include "model_config.hpp"

#include <algorithm>
#include <cctype>
#include <cstdlib>
#include <fstream>
#include <sstream>

namespace rembrandt {

const TomlValue* TomlValue::lookup(const std::string& key) const {
  for (const auto& kv : table)
    if (kv.first == key) return &kv.second;
  return nullptr;
}
TomlValue* TomlValue::lookup_mut(const std::string& key) {
  for (auto& kv : table)
    if (kv.first == key) return &kv.second;
  return nullptr;
}
double TomlValue::as_float() const {
  if (kind != Float) panic("toml: expected a float");
  return f;
}

namespace {

struct Cursor {
  const std::string& t;
  size_t p = 0;
  int line = 1;
  explicit Cursor(const std::string& text) : t(text) {}
  [[noreturn]] void fail(const std::string& why) const { panic("toml: line " + std::to_string(line) + ": " + why); }
  bool eof() const { return p >= t.size(); }
  char peek() const { return eof() ? '\0' : t[p]; }
  char get() {
    const char c = t[p++];
    if (c == '\n') ++line;
    return c;
  }
  void skip_inline_ws() { while (!eof() && (peek() == ' ' || peek() == '\t' || peek() == '\r')) ++p; }
  void skip_ws_comments_newlines() {
    for (;;) {
      skip_inline_ws();
      if (peek() == '#') { while (!eof() && peek() != '\n') ++p; }
      else if (peek() == '\n') get();
      else break;
    }
  }
  void end_of_line() {
    skip_inline_ws();
    if (peek() == '#') while (!eof() && peek() != '\n') ++p;
    if (!eof() && peek() != '\n') fail("unexpected characters after value");
  }
};

std::string parse_key(Cursor& c) {
  c.skip_inline_ws();
  std::string k;
  if (c.peek() == '"') {
    c.get();
    while (!c.eof() && c.peek() != '"') k += c.get();
    if (c.eof()) c.fail("unterminated key");
    c.get();
  } else {
    while (!c.eof() && (std::isalnum((unsigned char)c.peek()) || c.peek() == '_' || c.peek() == '-')) k += c.get();
  }
  if (k.empty()) c.fail("empty key");
  return k;
}

TomlValue parse_value(Cursor& c);

TomlValue parse_string(Cursor& c) {
  TomlValue v;
  v.kind = TomlValue::String;
  const char q = c.get();
  while (!c.eof() && c.peek() != q) {
    char ch = c.get();
    if (ch == '\n') c.fail("newline in string");
    if (ch == '\\' && q == '"') {
      if (c.eof()) c.fail("bad escape");
      const char e = c.get();
      switch (e) {
        case 'n': ch = '\n'; break;
        case 't': ch = '\t'; break;
        case '\\': ch = '\\'; break;
        case '"': ch = '"'; break;
        default: c.fail("unsupported escape");
      }
    }
    v.s += ch;
  }
  if (c.eof()) c.fail("unterminated string");
  c.get();
  return v;
}

TomlValue parse_number_or_bool(Cursor& c) {
  std::string tok;
  while (!c.eof() && (std::isalnum((unsigned char)c.peek()) || c.peek() == '+' || c.peek() == '-' || c.peek() == '.' ||
                      c.peek() == '_'))
    tok += c.get();
  TomlValue v;
  if (tok == "true" || tok == "false") {
    v.kind = TomlValue::Boolean;
    v.b = tok == "true";
    return v;
  }
  tok.erase(std::remove(tok.begin(), tok.end(), '_'), tok.end());
  if (tok.empty()) c.fail("expected a value");
  const bool is_float = tok.find_first_of(".eE") != std::string::npos;
  char* end = nullptr;
  if (is_float) {
    v.kind = TomlValue::Float;
    v.f = std::strtod(tok.c_str(), &end);
  } else {
    v.kind = TomlValue::Integer;
    v.i = std::strtoll(tok.c_str(), &end, 10);
  }
  if (!end || *end != '\0') c.fail("bad number '" + tok + "'");
  return v;
}

TomlValue parse_value(Cursor& c) {
  c.skip_inline_ws();
  const char ch = c.peek();
  if (ch == '"' || ch == '\'') return parse_string(c);
  if (ch == '[') {
    c.get();
    TomlValue v;
    v.kind = TomlValue::Array;
    for (;;) {
      c.skip_ws_comments_newlines();
      if (c.peek() == ']') { c.get(); break; }
      v.array.push_back(parse_value(c));
      c.skip_ws_comments_newlines();
      if (c.peek() == ',') { c.get(); continue; }
      if (c.peek() == ']') { c.get(); break; }
      c.fail("expected ',' or ']' in array");
    }
    return v;
  }
  if (ch == '{') {
    c.get();
    TomlValue v;
    v.kind = TomlValue::Table;
    for (;;) {
      c.skip_inline_ws();
      if (c.peek() == '}') { c.get(); break; }
      const std::string k = parse_key(c);
      c.skip_inline_ws();
      if (c.get() != '=') c.fail("expected '=' in inline table");
      v.table.emplace_back(k, parse_value(c));
      c.skip_inline_ws();
      if (c.peek() == ',') { c.get(); continue; }
      if (c.peek() == '}') { c.get(); break; }
      c.fail("expected ',' or '}' in inline table");
    }
    return v;
  }
  return parse_number_or_bool(c);
}

TomlValue* descend(TomlValue* root, const std::vector<std::string>& path, bool array_of_tables, Cursor& c) {
  TomlValue* cur = root;
  for (size_t i = 0; i < path.size(); ++i) {
    const bool last = i + 1 == path.size();
    TomlValue* next = cur->lookup_mut(path[i]);
    if (!next) {
      TomlValue nv;
      nv.kind = (last && array_of_tables) ? TomlValue::Array : TomlValue::Table;
      cur->table.emplace_back(path[i], nv);
      next = &cur->table.back().second;
    }
    if (last && array_of_tables) {
      if (next->kind != TomlValue::Array) c.fail("'" + path[i] + "' is not an array of tables");
      TomlValue t;
      t.kind = TomlValue::Table;
      next->array.push_back(t);
      return &next->array.back();
    }
    if (next->kind == TomlValue::Array) {
      if (next->array.empty()) c.fail("empty array of tables");
      next = &next->array.back();
    }
    if (next->kind != TomlValue::Table) c.fail("'" + path[i] + "' is not a table");
    cur = next;
  }
  return cur;
}

}  // namespace

TomlValue toml_parse(const std::string& text) {
  TomlValue root;
  root.kind = TomlValue::Table;
  TomlValue* cur = &root;
  Cursor c(text);
  for (;;) {
    c.skip_ws_comments_newlines();
    if (c.eof()) break;
    if (c.peek() == '[') {
      c.get();
      bool aot = false;
      if (c.peek() == '[') { c.get(); aot = true; }
      std::vector<std::string> path;
      for (;;) {
        path.push_back(parse_key(c));
        c.skip_inline_ws();
        if (c.peek() == '.') { c.get(); continue; }
        break;
      }
      if (c.get() != ']') c.fail("expected ']'");
      if (aot && c.get() != ']') c.fail("expected ']]'");
      c.end_of_line();
      cur = descend(&root, path, aot, c);
    } else {
      const std::string k = parse_key(c);
      c.skip_inline_ws();
      if (c.get() != '=') c.fail("expected '=' after key '" + k + "'");
      TomlValue v = parse_value(c);
      c.end_of_line();
      if (cur->lookup(k)) c.fail("duplicate key '" + k + "'");
      cur->table.emplace_back(k, v);
    }
  }
  return root;
}

static std::string read_file(const std::string& path) {
  std::ifstream f(path, std::ios::binary);
  if (!f) panic("failed to open config file: " + path);
  std::ostringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

// ---- .model -----------------------------------------------------------------------------------------
static size_t req_int(const TomlValue& node, const char* key) {
  const TomlValue* v = node.lookup(key);
  if (!v || v->kind != TomlValue::Integer || v->i < 0) panic(std::string("layer is missing integer field '") + key + "'");
  return (size_t)v->i;
}
static std::string req_str(const TomlValue& node, const char* key) {
  const TomlValue* v = node.lookup(key);
  if (!v || v->kind != TomlValue::String) panic(std::string("layer is missing string field '") + key + "'");
  return v->s;
}
static std::vector<std::string> str_list(const TomlValue& node, const char* one, const char* many) {
  std::vector<std::string> out;
  if (const TomlValue* v = node.lookup(one)) {
    if (v->kind != TomlValue::String) panic(std::string("'") + one + "' should be a string!");
    out.push_back(v->s);
  } else if (const TomlValue* vs = node.lookup(many)) {
    if (vs->kind != TomlValue::Array) panic(std::string("'") + many + "' should be an array!");
    for (const auto& e : vs->array) {
      if (e.kind != TomlValue::String) panic(std::string("'") + many + "' should be an array of strings!");
      out.push_back(e.s);
    }
  }
  return out;
}
static ActivationFunction parse_act(const std::string& s) {
  // src/config.rs:123-129 (the gen-1 "sigmoid" is the operator API's Logistic)
  if (s == "identity") return ActivationFunction::Identity;
  if (s == "rect") return ActivationFunction::Rect;
  if (s == "sigmoid") return ActivationFunction::Logistic;
  if (s == "tanh") return ActivationFunction::Tanh;
  panic("unimplemented act_func '" + s + "'");
}
static ParamsInit parse_init(const TomlValue& node) {
  const TomlValue* init = node.lookup("init_weights");
  if (!init || init->kind != TomlValue::Table) panic("layer is missing 'init_weights'");
  const std::string kind = req_str(*init, "kind");
  if (kind != "normal") panic("unimplemented init_weights kind '" + kind + "'");
  const TomlValue* mean = init->lookup("mean");
  const TomlValue* sd = init->lookup("std");
  if (!mean || !sd) panic("init_weights needs 'mean' and 'std'");
  (void)mean->as_float();
  return ParamsInit::MakeNormal((float)sd->as_float());
}

static Dims3 layer_out_dims(const LayerEntry& l) {
  if (l.type == "data") return {l.crop_width, l.crop_height, l.channels};
  if (l.type == "fully_conn") return {1, 1, l.out_channels};
  if (l.type == "conv2d") {
    // gen-1 extent max(0, in + 2*pad - size)/stride + 1  (src/layer.rs:1162-1168)
    auto f = [&](size_t in) {
      const long long t = (long long)in + 2 * (long long)l.conv_pad - (long long)l.conv_size;
      return (size_t)(std::max<long long>(0, t) / (long long)l.conv_stride + 1);
    };
    return {f(l.in_dims.w), f(l.in_dims.h), l.out_channels};
  }
  if (l.type == "pool") {
    // gen-1 extent max(0, in + 2*pad - size + stride - 1)/stride + 1  (src/layer.rs:1741-1747)
    auto f = [&](size_t in) {
      const long long t = (long long)in + 2 * (long long)l.pool_pad - (long long)l.pool_size + (long long)l.pool_stride - 1;
      return (size_t)(std::max<long long>(0, t) / (long long)l.pool_stride + 1);
    };
    return {f(l.in_dims.w), f(l.in_dims.h), l.in_dims.c};
  }
  if (l.type == "softmax_loss") return {1, 1, l.num_categories};
  return l.in_dims;  // local_res_norm, dropout keep the shape
}

ModelConfigFile ModelConfigFile::open(const std::string& path) { return parse(read_file(path)); }

ModelConfigFile ModelConfigFile::parse(const std::string& text) {
  const TomlValue root = toml_parse(text);
  const TomlValue* layer_nodes = root.lookup("layer");
  if (!layer_nodes || layer_nodes->kind != TomlValue::Array) panic("config file has no [[layer]] tables");
  ModelConfigFile out;
  std::map<std::string, size_t> name_ids;
  std::vector<size_t> prev_ids;
  bool have_prev = false;
  for (const TomlValue& node : layer_nodes->array) {
    LayerEntry l;
    l.names = str_list(node, "name", "names");
    if (l.names.empty()) panic("layer has neither 'name' nor 'names'");
    l.inputs = str_list(node, "input", "inputs");
    // input dims: channels of all inputs add up; width and height must agree (src/config.rs:58-100)
    std::vector<size_t> in_ids;
    if (have_prev && l.inputs.empty()) in_ids = prev_ids;
    for (const auto& n : l.inputs) {
      auto it = name_ids.find(n);
      if (it == name_ids.end()) panic("layer input '" + n + "' is not defined");
      in_ids.push_back(it->second);
    }
    l.in_dims = {0, 0, 0};
    for (size_t id : in_ids) {
      const Dims3 od = out.layers[id].out_dims;
      if (l.in_dims.w == 0) l.in_dims.w = od.w; else if (l.in_dims.w != od.w) panic("input widths disagree");
      if (l.in_dims.h == 0) l.in_dims.h = od.h; else if (l.in_dims.h != od.h) panic("input heights disagree");
      l.in_dims.c += od.c;
    }
    const TomlValue* ty = node.lookup("type");
    if (!ty || ty->kind != TomlValue::String) panic("'layer' missing 'type' field!");
    l.type = ty->s;
    if (l.type == "data") {
      if (have_prev) panic("data layer must come first");
      l.raw_width = req_int(node, "raw_width");
      l.raw_height = req_int(node, "raw_height");
      l.crop_width = req_int(node, "crop_width");
      l.crop_height = req_int(node, "crop_height");
      l.channels = req_int(node, "channels");
    } else if (l.type == "fully_conn") {
      l.out_channels = req_int(node, "out_channels");
      l.act_func = parse_act(req_str(node, "act_func"));
      l.init_weights = node.lookup("init_weights") ? parse_init(node) : ParamsInit::MakeNormal(0.01f);
    } else if (l.type == "conv2d") {
      l.conv_size = req_int(node, "conv_size");
      l.conv_stride = req_int(node, "conv_stride");
      l.conv_pad = req_int(node, "conv_pad");
      l.out_channels = req_int(node, "out_channels");
      l.act_func = parse_act(req_str(node, "act_func"));
      l.init_weights = parse_init(node);
      if (l.conv_stride == 0 || l.conv_size == 0) panic("conv2d needs positive conv_size and conv_stride");
    } else if (l.type == "pool") {
      l.pool_size = req_int(node, "pool_size");
      l.pool_stride = req_int(node, "pool_stride");
      l.pool_pad = req_int(node, "pool_pad");
      const std::string k = req_str(node, "pool_kind");
      if (k == "max") l.pool_kind = PoolOperation::Max;
      else if (k == "average") l.pool_kind = PoolOperation::Average;
      else panic("unimplemented pool_kind '" + k + "'");
      if (l.pool_stride == 0 || l.pool_size == 0) panic("pool needs positive pool_size and pool_stride");
    } else if (l.type == "local_res_norm") {
      l.cross_size = req_int(node, "cross_size");
      auto opt_float = [&](const char* key, float dflt) {
        const TomlValue* v = node.lookup(key);
        if (!v) return dflt;
        return v->kind == TomlValue::Integer ? (float)v->i : (float)v->as_float();  // `min_div = 2` in the examples
      };
      l.lrn_scale = opt_float("scale", 1.0e-4f);
      l.lrn_power = opt_float("power", 0.75f);
      l.lrn_min_div = opt_float("min_div", 2.0f);
    } else if (l.type == "dropout") {
      const TomlValue* r = node.lookup("drop_ratio");
      if (!r) panic("dropout layer is missing 'drop_ratio'");
      l.drop_ratio = (float)r->as_float();
    } else if (l.type == "softmax_loss") {
      l.num_categories = req_int(node, "num_categories");
      if (l.in_dims.len() != l.num_categories) panic("softmax_loss: input length != num_categories");
    } else {
      panic("unimplemented layer type '" + l.type + "'");
    }
    if (l.type != "data" && in_ids.empty()) panic("layer '" + l.names[0] + "' has no input");
    l.out_dims = layer_out_dims(l);
    // one entry per name (src/config.rs:229-262)
    prev_ids.clear();
    for (const auto& n : l.names) {
      LayerEntry e = l;
      e.names.assign(1, n);
      name_ids[n] = out.layers.size();
      prev_ids.push_back(out.layers.size());
      out.layers.push_back(e);
    }
    have_prev = true;
  }
  return out;
}

SequentialOperatorConfig ModelConfigFile::to_sequential_config() const {
  SequentialOperatorConfig cfg;
  for (const LayerEntry& l : layers) {
    if (l.type == "data") {
      // frames arrive at the raw size; a smaller crop becomes the input operator's Crop step
      Data3dOperatorConfig d = {{l.raw_width, l.raw_height, l.channels}, true, {}};
      if (l.crop_width > l.raw_width || l.crop_height > l.raw_height) panic("data layer: crop larger than the raw frame");
      if (l.crop_width != l.raw_width || l.crop_height != l.raw_height) {
        Data3dPreproc p;
        p.kind = Data3dPreproc::Crop;
        p.crop_width = l.crop_width;
        p.crop_height = l.crop_height;
        d.preprocs.push_back(p);
      }
      cfg.data3d(d);
    } else if (l.type == "conv2d") {
      cfg.conv2d({l.in_dims, l.conv_size, l.conv_stride, l.conv_pad, l.out_channels, l.act_func, l.init_weights});
    } else if (l.type == "pool") {
      cfg.pool2d({l.in_dims, l.pool_size, l.pool_stride, l.pool_pad, l.pool_kind, ActivationFunction::Identity, true});
    } else if (l.type == "fully_conn") {
      cfg.affine({l.in_dims.len(), l.out_channels, l.act_func, l.init_weights});
    } else if (l.type == "dropout") {
      cfg.dropout({l.in_dims.len(), l.drop_ratio});
    } else if (l.type == "local_res_norm") {
      cfg.local_res_norm({l.in_dims, l.cross_size, l.lrn_scale, l.lrn_power, l.lrn_min_div});
    } else if (l.type == "softmax_loss") {
      cfg.softmax_kl_loss({l.num_categories});
    } else {
      panic("layer type '" + l.type + "' has no operator in this build");
    }
  }
  if (!cfg.has_input) panic("model has no data layer");
  if (!cfg.has_loss) panic("model has no softmax_loss layer");
  return cfg;
}

// ---- .data ------------------------------------------------------------------------------------------
DatasetConfig DatasetConfig::open(const std::string& path) { return parse(read_file(path)); }

DatasetConfig DatasetConfig::parse(const std::string& text) {
  const TomlValue root = toml_parse(text);
  const TomlValue* data = root.lookup("dataset");
  if (!data || data->kind != TomlValue::Table) panic("[dataset] should be a table!");
  DatasetConfig out;
  for (const auto& kv : data->table) {
    const TomlValue& node = kv.second;
    if (node.kind != TomlValue::Table) panic("[dataset." + kv.first + "] should be a table!");
    DataSourceConfig c;
    c.source = req_str(node, "source");
    c.data_path = req_str(node, "data_path");
    if (const TomlValue* v = node.lookup("labels_path")) { c.labels_path = v->s; c.has_labels = true; }
    if (const TomlValue* v = node.lookup("labels2_path")) { c.labels2_path = v->s; c.has_labels2 = true; }
    out.datasets[kv.first] = c;
  }
  return out;
}

}  // namespace rembrandt
