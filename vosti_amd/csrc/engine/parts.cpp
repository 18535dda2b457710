#include "parts.h"

#include "../host/rules.h"

#include <dlfcn.h>

#include <algorithm>
#include <cmath>
#include <mutex>

namespace vosti {

// --------------------------------------------------------------------------------------- registry
namespace {
std::map<std::pair<std::string, std::string>, PartFactory>& part_registry() {
  static std::map<std::pair<std::string, std::string>, PartFactory> r;
  return r;
}
std::map<std::string, BlockFactory>& block_registry() {
  static std::map<std::string, BlockFactory> r;
  return r;
}
}  // namespace

void register_part(const std::string& category, const std::string& kind, PartFactory make) {
  part_registry()[{category, kind}] = std::move(make);
}
void register_block(const std::string& kind, BlockFactory make) { block_registry()[kind] = std::move(make); }
bool part_registered(const std::string& category, const std::string& kind) { return part_registry().count({category, kind}) > 0; }
bool block_registered(const std::string& kind) { return block_registry().count(kind) > 0; }

namespace {
std::string missing_in(const std::string& category, const PartSpec& p) {
  if (!part_registered(category, p.kind)) return category + " part '" + p.kind + "'";
  // Parts below a part: the name says the category ("q_norm", "k_norm": norms; "position"; "left_mixer": a mixer).
  auto ends_with = [](const std::string& s, const char* tail) {
    const size_t n = std::char_traits<char>::length(tail);
    return s.size() >= n && s.compare(s.size() - n, n, tail) == 0;
  };
  for (const auto& c : p.parts) {
    const std::string below = c.first == "position" ? "position" : (ends_with(c.first, "norm") ? "norm" : (ends_with(c.first, "mixer") ? "mixer" : ""));
    if (below.empty()) continue;
    const std::string m = missing_in(below, *c.second);
    if (!m.empty()) return m;
  }
  return "";
}
}  // namespace

std::string missing_part(const ModelSpec& spec) {
  std::string m = missing_in("embedding", *spec.embedding);
  if (m.empty()) m = missing_in("norm", *spec.final_norm);
  if (m.empty()) m = missing_in("head", *spec.head);
  for (const LayerSpec& l : spec.layers) {
    if (!m.empty()) break;
    if (!block_registered(l.block)) m = "block arrangement '" + l.block + "'";
    if (m.empty()) m = missing_in("mixer", *l.mixer);
    if (m.empty()) m = missing_in("feed_forward", *l.feed_forward);
    for (const auto& n : l.norms)
      if (m.empty()) m = missing_in("norm", *n.second);
  }
  return m;
}

void load_plugin(const std::string& path) {
  static std::mutex mutex;
  static std::map<std::string, void*> loaded;
  std::lock_guard<std::mutex> lock(mutex);
  if (loaded.count(path)) return;
  void* h = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
  if (!h) throw EngineError("cannot load the plugin " + path + ": " + dlerror());
  auto fn = reinterpret_cast<void (*)()>(dlsym(h, "vosti_plugin_register"));
  if (!fn) throw EngineError("the plugin " + path + " has no vosti_plugin_register()");
  register_standard_parts();
  register_builtin_architectures();
  fn();
  loaded[path] = h;
}

std::pair<Tensor, Tensor> PositionEncoding::apply(const Tensor& q, const Tensor& k, const Tensor& positions) {
  const Tensor *cos = cos_table(), *sin = sin_table(), *freq = angle_frequencies();
  if ((!cos || !sin) && !freq) throw EngineError("a position encoding needs tables of angles, frequencies or an apply() of its own");
  auto rotate = [&](const Tensor& x) {
    if (x.shape.size() != 3) throw EngineError("position encoding of " + x.describe() + ", expected [tokens, heads, head size]");
    const int64_t T = x.dim(0), n = x.dim(1), d = x.dim(2);
    if (freq && pairs_neighbours())
      return kernels.qkv_post_norm_angles_paired(x.view({T, n * d}), (int)n, 0, (int)d, nullptr, nullptr, 0, nullptr, nullptr, (int)d, 0.f, *freq, magnitude(),
                                                 true, positions, nullptr);
    if (freq) return kernels.qkv_post_angles(x.view({T, n * d}), (int)n, 0, (int)d, nullptr, nullptr, 0, *freq, magnitude(), positions, nullptr);
    return kernels.qkv_post(x.view({T, n * d}), (int)n, 0, (int)d, nullptr, nullptr, 0, nullptr, nullptr, 0.f, cos, sin, &positions, nullptr);
  };
  return {rotate(q), k.data ? rotate(k) : Tensor()};
}

void Norm::forward_scaled_add(const Tensor& y, const Tensor& base, Tensor& out, float mult, Tensor* rounded) {
  (void)y; (void)base; (void)out; (void)mult; (void)rounded;
  throw EngineError("this norm kind cannot add its scaled output to a 32-bit residual stream");
}

std::unique_ptr<Part> build_any_part(const std::string& category, const PartSpec& spec, Kernels& k) {
  auto it = part_registry().find({category, spec.kind});
  if (it == part_registry().end()) throw ConfigError("no " + category + " part of kind '" + spec.kind + "' in the native engine");
  return it->second(spec, k);
}

std::unique_ptr<Block> build_block(const LayerSpec& spec, Kernels& k) {
  auto it = block_registry().find(spec.block);
  if (it == block_registry().end()) throw ConfigError("no block arrangement of kind '" + spec.block + "' in the native engine");
  std::map<std::string, std::unique_ptr<Norm>> norms;
  for (const auto& n : spec.norms) norms[n.first] = build_part<Norm>("norm", *n.second, k);
  return it->second(k, build_part<Mixer>("mixer", *spec.mixer, k), build_part<FeedForward>("feed_forward", *spec.feed_forward, k),
                    std::move(norms), spec.block_numbers);
}

namespace {

Tensor need(std::map<std::string, Tensor>& tensors, const std::string& name) {
  auto it = tensors.find(name);
  if (it == tensors.end()) throw EngineError("a part was not given its tensor '" + name + "'");
  return it->second;
}

// Rows of several weights one under the other in one buffer, so that one launch projects them all.
Tensor stack_rows(const std::vector<Tensor>& pieces) {
  int64_t rows = 0;
  for (const Tensor& p : pieces) {
    if (p.shape.size() != 2 || p.dim(1) != pieces[0].dim(1) || p.dtype != pieces[0].dtype)
      throw EngineError("weights that are stacked must have one width and one type");
    rows += p.dim(0);
  }
  Tensor out;
  out.dtype = pieces[0].dtype;
  out.shape = {rows, pieces[0].dim(1)};
  out.owner = std::make_shared<DeviceBuffer>(out.bytes());
  out.data = out.owner->data();
  size_t at = 0;
  for (const Tensor& p : pieces) {
    hip_check(hipMemcpy(static_cast<char*>(out.data) + at, p.data, p.bytes(), hipMemcpyDeviceToDevice), "stacking weights");
    at += p.bytes();
  }
  return out;
}

Tensor zero_weight(std::vector<int64_t> shape, DType t) {
  Tensor out;
  out.dtype = t;
  out.shape = std::move(shape);
  out.owner = std::make_shared<DeviceBuffer>(out.bytes());
  out.data = out.owner->data();
  hip_check(hipMemset(out.data, 0, out.bytes()), "clearing a weight");
  return out;
}

// w [rows, cols] in the upper left corner of a zero matrix [rows_to, cols_to].
Tensor pad_matrix(const Tensor& w, int64_t rows_to, int64_t cols_to) {
  if (w.shape.size() != 2 || rows_to < w.dim(0) || cols_to < w.dim(1)) throw EngineError("a weight cannot be padded to a smaller size");
  if (rows_to == w.dim(0) && cols_to == w.dim(1)) return w;
  Tensor out = zero_weight({rows_to, cols_to}, w.dtype);
  const size_t e = (size_t)dtype_bytes(w.dtype);
  if (w.numel())
    hip_check(hipMemcpy2D(out.data, (size_t)cols_to * e, w.data, (size_t)w.dim(1) * e, (size_t)w.dim(1) * e, (size_t)w.dim(0), hipMemcpyDeviceToDevice),
              "padding a weight");
  return out;
}

// The rows of w [n * size, cols] as n blocks of size_to rows each, the new rows zero: a head's outputs padded.
Tensor pad_row_blocks(const Tensor& w, int64_t n, int64_t size, int64_t size_to) {
  const bool vec = w.shape.size() == 1;
  const Tensor m = vec ? w.view({w.dim(0), 1}) : w;
  if (m.shape.size() != 2 || m.dim(0) != n * size || size_to < size) throw EngineError("a weight of " + w.describe() + " is not " + std::to_string(n) + " blocks of " + std::to_string(size) + " rows");
  if (size_to == size) return w;
  Tensor out = zero_weight({n * size_to, m.dim(1)}, w.dtype);
  const size_t row = (size_t)m.dim(1) * dtype_bytes(w.dtype);
  for (int64_t b = 0; b < n; ++b)
    hip_check(hipMemcpy(static_cast<char*>(out.data) + (size_t)(b * size_to) * row, static_cast<const char*>(m.data) + (size_t)(b * size) * row,
                        (size_t)size * row, hipMemcpyDeviceToDevice),
              "padding a weight");
  return vec ? out.view({n * size_to}) : out;
}

// The columns of w [rows, n * size] as n blocks of size_to columns each, the new columns zero: a head's inputs padded.
Tensor pad_column_blocks(const Tensor& w, int64_t n, int64_t size, int64_t size_to) {
  if (w.shape.size() != 2 || w.dim(1) != n * size || size_to < size) throw EngineError("a weight of " + w.describe() + " is not " + std::to_string(n) + " blocks of " + std::to_string(size) + " columns");
  if (size_to == size) return w;
  Tensor out = zero_weight({w.dim(0), n * size_to}, w.dtype);
  const size_t e = (size_t)dtype_bytes(w.dtype);
  for (int64_t b = 0; b < n; ++b)
    hip_check(hipMemcpy2D(static_cast<char*>(out.data) + (size_t)(b * size_to) * e, (size_t)(n * size_to) * e,
                          static_cast<const char*>(w.data) + (size_t)(b * size) * e, (size_t)(n * size) * e, (size_t)size * e, (size_t)w.dim(0),
                          hipMemcpyDeviceToDevice),
              "padding a weight");
  return out;
}

int64_t round_up(int64_t n, int64_t to) { return (n + to - 1) / to * to; }

// h[t] = E[ids[t]], a row copy without scale (src/exec/dense_swiglu_model.rs:271-273).
class TokenEmbedding : public Embedding {
 public:
  TokenEmbedding(const PartSpec& s, Kernels& k) : Embedding(k), vocab_(s.integer("vocab_size")), hidden_(s.integer("hidden_size")) {}
  std::vector<ParamDecl> params() const override { return {{"weight", {vocab_, hidden_}}}; }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  Tensor forward(const Tensor& ids) override { return kernels.embedding(weight_, ids); }

 private:
  int64_t vocab_, hidden_;
  Tensor weight_;
};

// h[t] = E[ids[t]] + s(position of t), where s has sin(p * base^(-2i / width)) at entry 2i and the cosine of the same
// angle at entry 2i + 1.  The result is the residual stream in 32-bit, whatever the element type.  The frequencies are
// the 32-bit numbers that every host of these kernels computes for a rotation of the same base and width.
class SinusoidEmbedding : public Embedding {
 public:
  SinusoidEmbedding(const PartSpec& s, Kernels& k)
      : Embedding(k), vocab_(s.integer("vocab_size")), hidden_(s.integer("hidden_size")), base_(s.number("base")) {
    if (hidden_ % 2) throw ConfigError("sinusoidal positions need an even width, not " + std::to_string(hidden_));
  }
  std::vector<ParamDecl> params() const override { return {{"weight", {vocab_, hidden_}}}; }
  void load(std::map<std::string, Tensor>& t) override {
    weight_ = need(t, "weight");
    std::vector<float> inv((size_t)hidden_ / 2);
    rotary_inverse_frequencies(base_, (int)hidden_, inv.data());
    inv_freq_ = zero_weight({hidden_ / 2}, DType::F32);
    hip_check(hipMemcpy(inv_freq_.data, inv.data(), inv.size() * sizeof(float), hipMemcpyHostToDevice), "position frequencies");
  }
  Tensor forward(const Tensor&) override { throw EngineError("an embedding with positions needs the step's positions"); }
  Tensor forward(const Tensor& ids, StepContext& ctx) override { return kernels.embed_sinusoid(weight_, ids, ctx.positions, inv_freq_); }

 private:
  int64_t vocab_, hidden_;
  double base_;
  Tensor weight_, inv_freq_;
};

// h[t] = E[ids[t]] * scale, as the residual stream in 32-bit whatever the element type.
class ScaledEmbedding : public Embedding {
 public:
  ScaledEmbedding(const PartSpec& s, Kernels& k)
      : Embedding(k), vocab_(s.integer("vocab_size")), hidden_(s.integer("hidden_size")), scale_((float)s.number("scale", 1.0)) {}
  std::vector<ParamDecl> params() const override { return {{"weight", {vocab_, hidden_}}}; }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  Tensor forward(const Tensor& ids) override { return kernels.embed_scaled(weight_, ids, scale_); }

 private:
  int64_t vocab_, hidden_;
  float scale_;
  Tensor weight_;
};

// y = (x * rsqrt(mean(x^2) + eps)) * w in 32-bit (kernels/triton_kernels/rmsnorm.py:63-93); with a residual
// the norm sees the unrounded sum (kernels/triton_kernels/rmsnorm_residual.py:73-125).
class RMSNorm : public Norm {
 public:
  // offset: the weight that multiplies is offset + w (1 for a weight that is stored around zero, 0 by default).
  RMSNorm(const PartSpec& s, Kernels& k) : Norm(k), size_(s.integer("size")), eps_((float)s.number("eps")), offset_((float)s.number("offset", 0.0)) {}
  std::vector<ParamDecl> params() const override {
    if (offset_ != 0.f) return {{"weight", {size_}, true, true, -0.1, 0.1}};
    return {{"weight", {size_}, true, true, 0.9, 1.1}};
  }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  // Rows of a 32-bit residual stream are read as they are; the result is elements either way.
  Tensor forward(const Tensor& x) override {
    if (offset_ != 0.f || x.dtype != kernels.dtype()) return kernels.stream_norm(x, weight_, eps_, offset_);
    return kernels.rmsnorm(x, weight_, eps_);
  }
  Tensor forward_add(const Tensor& x, Tensor& residual) override {
    if (offset_ != 0.f) throw EngineError("a norm with a weight offset has no fused residual add in the element type");
    return kernels.add_rmsnorm(x, residual, weight_, eps_);
  }
  void forward_scaled_add(const Tensor& y, const Tensor& base, Tensor& out, float mult, Tensor* rounded) override {
    kernels.stream_norm_add(out, base, y, weight_, eps_, offset_, mult, rounded);
  }
  const Tensor* row_scale_weight() const override { return offset_ == 0.f ? &weight_ : nullptr; }
  float eps() const override { return eps_; }

 private:
  int64_t size_;
  float eps_, offset_;
  Tensor weight_;
};

// Half-rotation rotary encoding with tables (python/vosti_kernels/rotary.py:80-90 for the frequencies,
// :137-160 for the tables, kernels/triton_kernels/rope.py:78-123 for the rotation).  inv_freq[j] =
// 1 / theta^(2j / rotary_dim) is computed once on the host in 32-bit (rotary_inverse_frequencies, the one
// routine every host of these kernels uses); the angles, cosines and sines of every position are computed on
// the GPU in 32-bit and stored as elements.
class Rotary : public PositionEncoding {
 public:
  Rotary(const PartSpec& s, Kernels& k)
      : PositionEncoding(k), head_dim_(s.integer("head_dim")), rotary_dim_(s.integer("rotary_dim")), theta_(s.number("theta")),
        max_positions_(s.integer("max_positions")) {
    if (rotary_dim_ % 2 || rotary_dim_ <= 0 || rotary_dim_ > head_dim_)
      throw ConfigError("rotary width " + std::to_string(rotary_dim_) + " must be even and at most the head size " + std::to_string(head_dim_));
  }
  const Tensor* cos_table() override { return &ensure().first; }
  const Tensor* sin_table() override { return &ensure().second; }

 private:
  using Tables = std::pair<Tensor, Tensor>;
  const Tables& ensure() {
    if (tables_) return *tables_;
    // Layers with the same geometry share one pair of tables.
    static std::map<std::tuple<std::string, int64_t, double, int64_t>, std::shared_ptr<Tables>> shared;
    auto key = std::make_tuple(kernels.name(), rotary_dim_, theta_, max_positions_);
    auto it = shared.find(key);
    if (it == shared.end()) {
      const int64_t half = rotary_dim_ / 2;
      std::vector<float> inv(half);
      rotary_inverse_frequencies(theta_, (int)rotary_dim_, inv.data());
      DeviceBuffer inv_dev(half * sizeof(float));
      hip_check(hipMemcpy(inv_dev.data(), inv.data(), half * sizeof(float), hipMemcpyHostToDevice), "rotary frequencies");
      Tensor inv_t;
      inv_t.data = inv_dev.data();
      inv_t.dtype = DType::F32;
      inv_t.shape = {half};
      auto tables = std::make_shared<Tables>();
      for (Tensor* t : {&tables->first, &tables->second}) {
        t->dtype = kernels.dtype();
        t->shape = {max_positions_, half};
        t->owner = std::make_shared<DeviceBuffer>(t->bytes());
        t->data = t->owner->data();
      }
      kernels.rope_tables(tables->first, tables->second, inv_t);
      hip_check(hipStreamSynchronize(kernels.stream), "rotary tables");
      it = shared.emplace(key, tables).first;
    }
    tables_ = it->second;
    return *tables_;
  }
  int64_t head_dim_, rotary_dim_;
  double theta_;
  int64_t max_positions_;
  std::shared_ptr<Tables> tables_;
};

// The same half-rotation with angles that are computed where they are used, in 32-bit, and frequencies whose long
// wavelengths are stretched (rotary_stretched_frequencies has the rule): numbers rotary_dim, theta and, for a stretch,
// factor, original, fast, slow.  Cosine and sine are multiplied by 0.1 ln(factor) + 1.  linear_factor instead of factor:
// every frequency is divided by it and nothing else changes (rotary_linear_frequencies).  neighbours 1: a pair is a head's
// elements 2c and 2c + 1 instead of c and c + half.
class RotaryStretched : public PositionEncoding {
 public:
  RotaryStretched(const PartSpec& s, Kernels& k) : PositionEncoding(k), head_dim_(s.integer("head_dim")), rotary_dim_(s.integer("rotary_dim")) {
    if (rotary_dim_ % 2 || rotary_dim_ <= 0 || rotary_dim_ > head_dim_)
      throw ConfigError("rotary width " + std::to_string(rotary_dim_) + " must be even and at most the head size " + std::to_string(head_dim_));
    std::vector<float> f((size_t)rotary_dim_ / 2);
    neighbours_ = s.integer("neighbours", 0) != 0;
    const double linear = s.number("linear_factor", 0.0);
    if (linear < 0 || (linear > 0 && s.number("factor", 0.0) > 0)) throw ConfigError("a rotation is stretched by 'factor' or by 'linear_factor', not both");
    if (linear > 0) rotary_linear_frequencies(s.number("theta"), (int)rotary_dim_, linear, f.data());
    else
      mag_ = rotary_stretched_frequencies(s.number("theta"), (int)rotary_dim_, s.number("factor", 0.0), s.number("original", 1.0), s.number("fast", 1.0),
                                          s.number("slow", 1.0), f.data());
    freq_ = zero_weight({rotary_dim_ / 2}, DType::F32);
    hip_check(hipMemcpy(freq_.data, f.data(), f.size() * sizeof(float), hipMemcpyHostToDevice), "rotation frequencies");
  }
  const Tensor* angle_frequencies() override { return &freq_; }
  float magnitude() override { return mag_; }
  bool pairs_neighbours() const override { return neighbours_; }

 private:
  int64_t head_dim_, rotary_dim_;
  float mag_ = 1.f;
  bool neighbours_ = false;
  Tensor freq_;
};

// The attention kernels work on items: a single decoded token, or up to item_rows() consecutive rows of a
// sequence that brings several tokens.  The item lists are the same for every attention layer of a step.
struct AttentionItems {
  HostArray prefill, decode;
  int decode_bound = 0, nseg = 0;
};

// The items of a step, derived once a step and shared by every mixer that runs the paged attention kernels.
AttentionItems& attention_items(Kernels& kernels, HostStep& step) {
  auto it = step.memo.find("attention.items");
  if (it != step.memo.end()) return *static_cast<AttentionItems*>(it->second.get());
  auto m = std::make_shared<AttentionItems>();
  const int rows = kernels.item_rows();
  int decode_keys = 0;
  for (size_t s = 0; s < step.q_lens.size(); ++s) {
    if (step.q_lens[s] == 1) {
      m->decode.data.push_back((int32_t)s);
      m->decode.data.push_back(0);
      decode_keys = std::max(decode_keys, step.k_lens[s]);
    } else {
      for (int off = 0; off < step.q_lens[s]; off += rows) {
        m->prefill.data.push_back((int32_t)s);
        m->prefill.data.push_back(off);
      }
    }
  }
  m->prefill.shape = {(int64_t)m->prefill.data.size() / 2, 2};
  m->decode.shape = {(int64_t)m->decode.data.size() / 2, 2};
  // Recorded launches must cover every length that the tables can hold.
  m->decode_bound = step.frozen ? step.k_len_bound : decode_keys;
  m->nseg = (m->decode_bound + kernels.segment_keys() - 1) / kernels.segment_keys();
  step.memo["attention.items"] = m;
  return *m;
}

// Causal grouped-query attention over the paged cache (src/exec/dense_swiglu_decoder.rs:171-367): QKV
// projection without bias, per-head norm of q and k, rotary encoding, store of k and v, attention, output
// projection.  window > 0 limits a query to that many last keys.  q_norm, k_norm and position are parts of
// their own; when they are weighted row scales and a rotation by tables the three steps between the projections
// run as one launch.
//
// Further parameters, all optional: value_dim (the values' head size, where it differs from the keys'), bias (q, k
// and v projections with biases), softcap (score <- softcap * tanh(score / softcap)), keep_first (with a window: the
// first keys of a sequence stay visible), sink (a learned number per head whose exponential joins the softmax's
// denominator), exact_weights (the probabilities meet the values in 32-bit), own_kv 0 (the layer has no key and
// value projections: it always reads another execution's cache), block (positions are cut into blocks of this many from
// the sequence's start, and a query sees the earlier keys of its own block only; sink 2 is the constant 0 as every
// head's sink), output_gate (the heads' outputs are multiplied element by element with sigmoid(W_gate h), a projection of
// the mixer's own input, before the output projection).  The cache and the kernels see one head size: the
// larger of the two, rounded up to 16; the shorter of keys and values is padded with zeros in the weights, so that
// the projections write the padding and the output projection ignores it.
class Attention : public Mixer {
 public:
  Attention(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), nq_((int)s.integer("num_heads")), nkv_((int)s.integer("num_kv_heads")),
        dk_((int)s.integer("head_dim")), dv_((int)s.integer("value_dim", s.integer("head_dim"))), scale_((float)s.number("scale")),
        window_((int)s.integer("window", 0)), keep_((int)s.integer("keep_first", 0)), softcap_((float)s.number("softcap", 0.0)),
        bias_(s.integer("bias", 0) != 0), sink_((int)s.integer("sink", 0)), exact_(s.integer("exact_weights", 0) != 0),
        own_kv_(s.integer("own_kv", 1) != 0), block_((int)s.integer("block", 0)), gate_(s.integer("output_gate", 0) != 0) {
    d_ = (int)round_up(std::max(dk_, dv_), 16);
    if (nq_ % nkv_) throw ConfigError(std::to_string(nq_) + " heads are not a multiple of " + std::to_string(nkv_) + " kv heads");
    if (dk_ < 1 || dv_ < 1 || d_ > 256)
      throw ConfigError("head sizes " + std::to_string(dk_) + " and " + std::to_string(dv_) + ": the attention kernels take up to 256");
    if (window_ == 0) keep_ = 0;
    if (block_ < 0 || (block_ > 0 && window_ > 0)) throw ConfigError("attention: blocks of positions and a window exclude each other");
    if (sink_ < 0 || sink_ > 2) throw ConfigError("attention: 'sink' is 0 (none), 1 (a learned number per head) or 2 (the constant 0)");
    if (const PartSpec* p = s.part("q_norm")) q_norm_ = build_part<Norm>("norm", *p, k);
    if (const PartSpec* p = s.part("k_norm")) k_norm_ = build_part<Norm>("norm", *p, k);
    if (const PartSpec* p = s.part("position")) position_ = build_part<PositionEncoding>("position", *p, k);
    if (bias_ && (q_norm_ || k_norm_ || position_))
      throw ConfigError("attention: biases are not built together with head norms or a position encoding");
  }
  // The kernel with capped scores serves every one of these.
  bool capped() const { return softcap_ > 0.f || keep_ > 0 || sink_ || exact_ || block_ > 0; }
  std::vector<ParamDecl> params() const override {
    std::vector<ParamDecl> p = {{"q_proj.weight", {(int64_t)nq_ * dk_, hidden_}}, {"o_proj.weight", {hidden_, (int64_t)nq_ * dv_}}};
    if (own_kv_) {
      p.push_back({"k_proj.weight", {(int64_t)nkv_ * dk_, hidden_}});
      p.push_back({"v_proj.weight", {(int64_t)nkv_ * dv_, hidden_}});
    }
    if (bias_) {
      p.push_back({"q_proj.bias", {(int64_t)nq_ * dk_}});
      if (own_kv_) {
        p.push_back({"k_proj.bias", {(int64_t)nkv_ * dk_}});
        p.push_back({"v_proj.bias", {(int64_t)nkv_ * dv_}});
      }
    }
    if (sink_ == 1) {
      ParamDecl sinks{"sinks", {(int64_t)nq_}, true, true, -1.0, 1.0};
      p.push_back(sinks);
    }
    if (gate_) p.push_back({"gate_proj.weight", {(int64_t)nq_ * dv_, hidden_}});
    return p;
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c;
    if (q_norm_) c.emplace_back("q_norm", q_norm_.get());
    if (k_norm_) c.emplace_back("k_norm", k_norm_.get());
    if (position_) c.emplace_back("position", position_.get());
    return c;
  }
  void load(std::map<std::string, Tensor>& t) override {
    // One launch projects q, k and v (kernels/triton_kernels/qkv_matmul.py:108-211); rows of the fused
    // weight are q's, then k's, then v's.
    std::vector<Tensor> rows = {pad_row_blocks(need(t, "q_proj.weight"), nq_, dk_, d_)};
    if (own_kv_) {
      rows.push_back(pad_row_blocks(need(t, "k_proj.weight"), nkv_, dk_, d_));
      rows.push_back(pad_row_blocks(need(t, "v_proj.weight"), nkv_, dv_, d_));
    }
    // The output gate's rows follow the heads', so that the steps between the projections read the heads where they were.
    if (gate_) rows.push_back(pad_row_blocks(need(t, "gate_proj.weight"), nq_, dv_, d_));
    w_qkv_ = rows.size() > 1 ? stack_rows(rows) : rows[0];
    w_o_ = pad_column_blocks(need(t, "o_proj.weight"), nq_, dv_, d_);
    if (bias_) {
      std::vector<Tensor> b = {pad_row_blocks(need(t, "q_proj.bias"), nq_, dk_, d_)};
      if (own_kv_) {
        b.push_back(pad_row_blocks(need(t, "k_proj.bias"), nkv_, dk_, d_));
        b.push_back(pad_row_blocks(need(t, "v_proj.bias"), nkv_, dv_, d_));
      }
      for (Tensor& piece : b) piece = piece.view({piece.numel(), 1});
      b_qkv_ = b.size() > 1 ? stack_rows(b) : b[0];
      b_qkv_ = b_qkv_.view({b_qkv_.numel()});
    }
    if (sink_ == 1) sinks_ = need(t, "sinks");
    if (sink_ == 2) sinks_ = zero_weight({(int64_t)nq_}, DType::F32);      // exp(0) = 1 joins every head's denominator
  }
  // Head norms, rotation and cache store run as one launch when the norms are weighted row scales with one eps
  // and the position encoding is a rotation by tables; any other kind runs through its own methods, step by step.
  // Asked when the sub-parts have their tensors (a norm's weight, a rotation's tables).
  bool fused() {
    for (Norm* n : {q_norm_.get(), k_norm_.get()})
      if (n && !n->row_scale_weight()) return false;
    if (q_norm_ && k_norm_ && q_norm_->eps() != k_norm_->eps()) return false;
    return !position_ || position_->cos_table() != nullptr || position_->angle_frequencies() != nullptr;
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::Pages;
    n.num_kv_heads = nkv_;
    n.head_dim = d_;
    n.window = window_;
    n.keep_first = keep_;
    return n;
  }
  const char* step_inputs_key() const override { return "attention.items"; }

  AttentionItems& items(HostStep& step) { return attention_items(kernels, step); }
  void step_inputs(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) override {
    AttentionItems& m = items(step);
    out.emplace_back("attention.prefill_items", m.prefill);
    out.emplace_back("attention.decode_items", m.decode);
  }
  // Workspace with which the two projections of T rows take their faster route, where there is one.
  int64_t gemm_floats(int64_t T) const {
    return std::max(kernels.gemm_workspace_floats(T, (int64_t)(nq_ + 2 * nkv_ + (gate_ ? nq_ : 0)) * d_, hidden_),
                    kernels.gemm_workspace_floats(T, hidden_, (int64_t)nq_ * d_));
  }
  int64_t workspace_floats(HostStep& step) override {
    AttentionItems& m = items(step);
    int64_t T = 0;
    for (int q : step.q_lens) T += q;
    int64_t need = gemm_floats(T);
    if (m.decode.shape[0]) need = std::max(need, kernels.attn_scratch_floats((int)m.decode.shape[0], nq_, d_, m.nseg));
    return need;
  }

  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::Pages) throw EngineError("attention was handed a cache entry without pages");
    Kernels& k = kernels;
    const int64_t T = x.dim(0);
    GroupTables& tables = ctx.groups.at(cache.group);
    // Without a cache of its own the keys and values are an earlier execution's: only q is projected.
    // The projections, the attention of decoded tokens and the next projection use the step's workspace one
    // after the other.
    const int64_t gf = gemm_floats(T);
    Tensor ws_t;
    if (gf) ws_t = ctx.workspace(gf);
    const Tensor* ws = gf ? &ws_t : nullptr;
    if (cache.writable && !own_kv_) throw EngineError("an attention layer without key and value projections was given a cache to write");
    // Rows of the stacked weight: q, then k and v (where the layer has them), then the output gate.  An execution that
    // reads another's cache projects q and the gate alone; without a gate, q's rows are the first of the weight.
    const int64_t heads_w = (int64_t)(nq_ + (cache.writable ? 2 * nkv_ : 0)) * d_;
    Tensor qkv_all;
    if (cache.writable || !own_kv_) qkv_all = k.gemm(x, w_qkv_, ws);
    else if (!gate_) qkv_all = k.gemm(x, w_qkv_.rows(0, (int64_t)nq_ * d_), ws);
    else throw EngineError("an attention layer with an output gate and projections of its own cannot read another execution's cache");
    const bool padded_norm = d_ != dk_ && (q_norm_ || k_norm_);
    const bool norm_angles = position_ && position_->angle_frequencies() && (q_norm_ || k_norm_) && fused();
    if (padded_norm && !norm_angles) throw ConfigError("attention: head norms on padded head sizes are built for rotations by computed angles only");
    // The kernels between the projections take rows of exactly the heads' width, except the one that says otherwise.
    const Tensor qkv = (qkv_all.dim(1) == heads_w || norm_angles) ? qkv_all : k.columns(qkv_all, 0, heads_w);
    Tensor q;
    if (norm_angles) {
      const Norm* en = q_norm_ ? q_norm_.get() : k_norm_.get();
      q = k.qkv_post_norm_angles_paired(qkv, nq_, cache.writable ? nkv_ : 0, d_, &cache.k, &cache.v, cache.page_size,
                                        q_norm_ ? q_norm_->row_scale_weight() : nullptr, k_norm_ && cache.writable ? k_norm_->row_scale_weight() : nullptr,
                                        dk_, en->eps(), *position_->angle_frequencies(), position_->magnitude(), position_->pairs_neighbours(),
                                        ctx.positions, &tables.slots);
    } else if (position_ && position_->pairs_neighbours()) {
      throw ConfigError("attention: a rotation of neighbouring pairs is built together with head norms");
    } else if (bias_) {
      const int64_t bw = (int64_t)(nq_ + (cache.writable ? 2 * nkv_ : 0)) * d_;
      q = k.qkv_post_bias(qkv, nq_, cache.writable ? nkv_ : 0, d_, &cache.k, &cache.v, cache.page_size, &tables.slots, b_qkv_.rows(0, bw));
    } else if (position_ && position_->angle_frequencies() && !q_norm_ && !k_norm_) {
      q = k.qkv_post_angles(qkv, nq_, cache.writable ? nkv_ : 0, d_, &cache.k, &cache.v, cache.page_size, *position_->angle_frequencies(),
                            position_->magnitude(), ctx.positions, &tables.slots);
    } else if (fused() && !(position_ && position_->angle_frequencies())) {
      const Norm* en = q_norm_ ? q_norm_.get() : k_norm_.get();
      q = k.qkv_post(qkv, nq_, cache.writable ? nkv_ : 0, d_, &cache.k, &cache.v, cache.page_size,
                     q_norm_ ? q_norm_->row_scale_weight() : nullptr, k_norm_ ? k_norm_->row_scale_weight() : nullptr,
                     en ? en->eps() : 0.f, position_ ? position_->cos_table() : nullptr,
                     position_ ? position_->sin_table() : nullptr, &ctx.positions, &tables.slots);
    } else {
      q = unfused(qkv, ctx, cache, tables);
    }
    Tensor out = k.empty(q.shape);
    AttentionItems& m = items(*ctx.host);
    const Tensor& prefill_items = ctx.inputs.at("attention.prefill_items");
    const Tensor& decode_items = ctx.inputs.at("attention.decode_items");
    const Tensor* sinks = sink_ ? &sinks_ : nullptr;
    if (prefill_items.dim(0)) {
      if (capped())
        k.paged_attention_capped(out, q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, prefill_items, 0, scale_, window_, keep_,
                                 softcap_, sinks, ctx.host->k_len_bound, 0, nullptr, block_);
      else
        k.paged_attention(out, q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, prefill_items, 0, scale_, window_,
                          ctx.host->k_len_bound, 0, nullptr);
    }
    if (decode_items.dim(0)) {
      const Tensor scratch = ctx.workspace(k.attn_scratch_floats((int)decode_items.dim(0), nq_, d_, m.nseg));
      if (capped())
        k.paged_attention_capped(out, q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, decode_items, 1, scale_, window_, keep_,
                                 softcap_, sinks, m.decode_bound, m.nseg, &scratch, block_);
      else
        k.paged_attention(out, q, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, decode_items, 1, scale_, window_,
                          m.decode_bound, m.nseg, &scratch);
    }
    Tensor heads = out.view({T, (int64_t)nq_ * d_});
    if (gate_) k.gate_mul(heads, qkv_all, heads_w, 0);
    return k.gemm(heads, w_o_, ws);
  }

 private:
  // Norm, position encoding and store as separate steps, each sub-part through its own methods.
  Tensor unfused(const Tensor& qkv, StepContext& ctx, CacheEntry& cache, GroupTables& tables) {
    Kernels& k = kernels;
    const int64_t T = qkv.dim(0), qw = (int64_t)nq_ * d_, kw = (int64_t)nkv_ * d_;
    Tensor q = k.columns(qkv, 0, qw).view({T, nq_, d_});
    if (q_norm_) q = q_norm_->forward(q);
    if (!cache.writable) {
      if (position_) q = position_->apply(q, Tensor(), ctx.positions).first;
      return q;
    }
    Tensor kk = k.columns(qkv, qw, kw).view({T, nkv_, d_});
    if (k_norm_) kk = k_norm_->forward(kk);
    if (position_) std::tie(q, kk) = position_->apply(q, kk, ctx.positions);
    Tensor kv = k.empty({T, 2 * kw});
    k.copy_columns(kv, 0, kk.view({T, kw}), 0, kw);
    k.copy_columns(kv, kw, qkv, qw + kw, kw);
    k.qkv_post(kv, 0, nkv_, d_, &cache.k, &cache.v, cache.page_size, nullptr, nullptr, 0.f, nullptr, nullptr, nullptr, &tables.slots);
    return q;
  }

  int64_t hidden_;
  int nq_, nkv_, dk_, dv_, d_ = 0;   // d_: the head size of the cache and the kernels
  float scale_;
  int window_, keep_;
  float softcap_;
  bool bias_;
  int sink_;                          // 0: none, 1: a learned number per head, 2: the constant 0
  bool exact_, own_kv_;
  int block_;                         // > 0: a row sees the keys of its own block of this many positions only
  bool gate_;                         // the heads' outputs times sigmoid(W_gate h)
  std::unique_ptr<Norm> q_norm_, k_norm_;
  std::unique_ptr<PositionEncoding> position_;
  Tensor w_qkv_, w_o_, b_qkv_, sinks_;
};

// down(silu(gate(x)) * up(x)) without biases (src/exec/dense_swiglu_decoder.rs:396-438); gate and up are one
// projection whose output is rounded before the activation
// (python/vosti_kernels/model_families/qwen3/loader.py:55-58, kernels/triton_kernels/silu_mul.py:64-87).
class SwiGLU : public FeedForward {
 public:
  SwiGLU(const PartSpec& s, Kernels& k) : FeedForward(k), hidden_(s.integer("hidden_size")), inter_(s.integer("intermediate_size")) {}
  std::vector<ParamDecl> params() const override {
    return {{"gate_proj.weight", {inter_, hidden_}}, {"up_proj.weight", {inter_, hidden_}}, {"down_proj.weight", {hidden_, inter_}}};
  }
  void load(std::map<std::string, Tensor>& t) override {
    // An intermediate size that is no multiple of 8 is padded with zero rows (and zero columns of the down projection):
    // the products' reduction axis must be whole 16-byte vectors, and silu(0) * 0 adds nothing.
    const int64_t padded = round_up(inter_, 8);
    w_gate_up_ = stack_rows({pad_matrix(need(t, "gate_proj.weight"), padded, hidden_), pad_matrix(need(t, "up_proj.weight"), padded, hidden_)});
    w_down_ = pad_matrix(need(t, "down_proj.weight"), hidden_, padded);
    inter_run_ = padded;
  }
  int64_t gemm_floats(int64_t T) const {
    const int64_t inter = inter_run_ ? inter_run_ : inter_;
    return std::max(kernels.gemm_workspace_floats(T, 2 * inter, hidden_, true), kernels.gemm_workspace_floats(T, hidden_, inter));
  }
  int64_t workspace_floats(HostStep& step) override {
    int64_t T = 0;
    for (int q : step.q_lens) T += q;
    return gemm_floats(T);
  }
  Tensor forward(const Tensor& x, StepContext& ctx) override {
    const int64_t n = gemm_floats(x.dim(0));
    Tensor ws;
    if (n) ws = ctx.workspace(n);
    return kernels.gemm(kernels.gemm_swiglu(x, w_gate_up_, n ? &ws : nullptr), w_down_, n ? &ws : nullptr);
  }

 private:
  int64_t hidden_, inter_, inter_run_ = 0;   // inter_run_: the intermediate size as the kernels see it
  Tensor w_gate_up_, w_down_;
};

// x += mixer(norm(x)); x += ffn(norm(x)), carried as (hidden, residual) so that each add runs inside the
// next norm (src/exec/dense_swiglu_decoder.rs:556-615 first layer, :740-813 others).
class PreNormBlock : public Block {
 public:
  PreNormBlock(Kernels& k, std::unique_ptr<Mixer> mixer, std::unique_ptr<FeedForward> ffn, std::map<std::string, std::unique_ptr<Norm>> norms)
      : Block(k), mixer_(std::move(mixer)), ffn_(std::move(ffn)), norms_(std::move(norms)) {
    for (const char* n : {"input", "post_mixer"})
      if (!norms_.count(n)) throw ConfigError(std::string("a prenorm block needs the norms 'input' and 'post_mixer'; missing: ") + n);
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c = {{"mixer", mixer_.get()}, {"feed_forward", ffn_.get()}};
    for (auto& n : norms_) c.emplace_back("norms." + n.first, n.second.get());
    return c;
  }
  Mixer& mixer() override { return *mixer_; }
  std::pair<Tensor, Tensor> forward(const Tensor& hidden, Tensor residual, StepContext& ctx, CacheEntry& cache) override {
    Tensor normed;
    if (residual.data == nullptr) {
      residual = hidden;
      normed = norms_["input"]->forward(hidden);
    } else {
      normed = norms_["input"]->forward_add(hidden, residual);
    }
    const Tensor mixed = mixer_->forward(normed, ctx, cache);
    normed = norms_["post_mixer"]->forward_add(mixed, residual);
    return {ffn_->forward(normed, ctx), residual};
  }

 private:
  std::unique_ptr<Mixer> mixer_;
  std::unique_ptr<FeedForward> ffn_;
  std::map<std::string, std::unique_ptr<Norm>> norms_;
};

// logits = x W^T without bias (src/exec/dense_swiglu_model.rs:976-984).  A head tied to the embedding is this
// same part: the architecture gives its weight the embedding table's tensor name, and the model hands both
// parts the one tensor (python/vosti_kernels/model_families/qwen3/physical.py:131-134).
class LinearHead : public Head {
 public:
  // softcap > 0: logits <- softcap * tanh(logits / softcap).
  LinearHead(const PartSpec& s, Kernels& k)
      : Head(k), vocab_(s.integer("vocab_size")), hidden_(s.integer("hidden_size")), softcap_((float)s.number("softcap", 0.0)) {}
  std::vector<ParamDecl> params() const override { return {{"weight", {vocab_, hidden_}}}; }
  void load(std::map<std::string, Tensor>& t) override { weight_ = need(t, "weight"); }
  Tensor forward(const Tensor& x) override {
    Tensor logits = kernels.gemm(x, weight_);
    if (softcap_ > 0.f) kernels.softcap(logits, softcap_);
    return logits;
  }

 private:
  int64_t vocab_, hidden_;
  float softcap_;
  Tensor weight_;
};

// Which sequence of the step every token belongs to: what a short convolution over a step's rows needs.
void token_sequences(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) {
  HostArray a;
  for (size_t s = 0; s < step.q_lens.size(); ++s) a.data.insert(a.data.end(), (size_t)step.q_lens[s], (int32_t)s);
  a.shape = {(int64_t)a.data.size()};
  out.emplace_back("delta.token_seq", std::move(a));
}

// The gated delta rule with one decay per head and key channel.  For the mixer's input h:
//   q = W_q h, k = W_k h (kv heads x key size), v = W_v h (heads x value size), each through a short causal
//   convolution per channel (taps [channels, K], the last tap the current token's, zeros before a sequence's start)
//   and silu; q and k become unit vectors per head (x / sqrt(sum(x^2) + unit_eps)), q times key size^(-1/2);
//   beta = sigmoid(W_b h) per head; g = exp(-exp(A_log[head]) * softplus(W_a2 (W_a1 h) + dt_bias)) per head and key
//   channel; per head, token by token:  S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
//   y = o / sqrt(mean(o^2) + eps) * w_norm * sigmoid(W_g2 (W_g1 h)) per head; out = W_o y.
// A request's state slot holds the heads' S in 32-bit and the last K - 1 inputs of the three convolutions.  The six
// input projections are one launch (their weights stacked, each section padded to a multiple of 8 rows with zero
// rows, so that the low-rank pairs' second halves read their columns in place); conv, norms, decays, recurrence and
// read-out are kernels of delta.hip, all in 32-bit.
class ChannelDelta : public Mixer {
 public:
  ChannelDelta(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), H_((int)s.integer("num_heads")), G_((int)s.integer("num_kv_heads")),
        d_((int)s.integer("key_dim")), dv_((int)s.integer("value_dim")), taps_((int)s.integer("conv_taps")),
        decay_rank_(s.integer("decay_rank", 0)), gate_rank_(s.integer("gate_rank", 0)), eps_((float)s.number("eps")),
        unit_eps_((float)s.number("unit_eps", 1e-6)) {
    if (H_ % G_) throw ConfigError(std::to_string(H_) + " heads are not a multiple of " + std::to_string(G_) + " kv heads");
    if (taps_ < 1 || taps_ > 17) throw ConfigError("a short convolution of " + std::to_string(taps_) + " taps: 1 to 17 are built");
    qk_ = round_up((int64_t)G_ * d_, 8);
    v_ = round_up((int64_t)H_ * dv_, 8);
    channels_ = 2 * qk_ + v_;
  }
  std::vector<ParamDecl> params() const override {
    const int64_t qk = (int64_t)G_ * d_, v = (int64_t)H_ * dv_, hd = (int64_t)H_ * d_;
    // 0: the rank is whatever the stored tensors have.
    const int64_t ra = decay_rank_ > 0 ? decay_rank_ : -1, rg = gate_rank_ > 0 ? gate_rank_ : -1;
    auto uniform = [](const char* name, std::vector<int64_t> shape, double lo, double hi) {
      ParamDecl p{name, std::move(shape), true, true, lo, hi};
      return p;
    };
    ParamDecl taps_q{"q_conv.weight", {qk, taps_}}, taps_k{"k_conv.weight", {qk, taps_}}, taps_v{"v_conv.weight", {v, taps_}};
    taps_q.p0 = taps_k.p0 = taps_v.p0 = 0.3;
    ParamDecl q{"q_proj.weight", {qk, hidden_}}, kk{"k_proj.weight", {qk, hidden_}}, vv{"v_proj.weight", {v, hidden_}};
    q.p0 = kk.p0 = vv.p0 = 0.1;
    ParamDecl a1{"decay_down.weight", {ra, hidden_}}, a2{"decay_up.weight", {hd, ra}}, g1{"gate_down.weight", {rg, hidden_}}, g2{"gate_up.weight", {v, rg}};
    a1.free_size = a2.free_size = g1.free_size = g2.free_size = std::max<int64_t>(8, hidden_ / 16);
    return {q, taps_q, kk, taps_k, vv, taps_v, {"beta_proj.weight", {(int64_t)H_, hidden_}}, uniform("A_log", {(int64_t)H_}, -1.0, 1.0),
            uniform("out_norm.weight", {(int64_t)dv_}, 0.9, 1.1), a1, a2, uniform("dt_bias", {hd}, -1.0, 1.0), g1, g2,
            {"o_proj.weight", {hidden_, v}}};
  }
  void load(std::map<std::string, Tensor>& t) override {
    const Tensor a1 = need(t, "decay_down.weight"), a2 = need(t, "decay_up.weight"), g1 = need(t, "gate_down.weight"), g2 = need(t, "gate_up.weight");
    if (a1.dim(0) != a2.dim(1) || g1.dim(0) != g2.dim(1))
      throw EngineError("the delta rule's low-rank projections do not fit each other: " + a1.describe() + " with " + a2.describe() + ", " +
                        g1.describe() + " with " + g2.describe());
    const int64_t ra = round_up(a1.dim(0), 8), rg = round_up(g1.dim(0), 8), nb = round_up(H_, 8);
    const int64_t qk = (int64_t)G_ * d_, v = (int64_t)H_ * dv_;
    w_in_ = stack_rows({pad_matrix(need(t, "q_proj.weight"), qk_, hidden_), pad_matrix(need(t, "k_proj.weight"), qk_, hidden_),
                        pad_matrix(need(t, "v_proj.weight"), v_, hidden_), pad_matrix(need(t, "beta_proj.weight"), nb, hidden_),
                        pad_matrix(a1, ra, hidden_), pad_matrix(g1, rg, hidden_)});
    beta_col_ = channels_;
    decay_col_ = beta_col_ + nb;
    gate_col_ = decay_col_ + ra;
    w_decay_up_ = pad_matrix(a2, a2.dim(0), ra);
    w_gate_up_ = pad_matrix(g2, g2.dim(0), rg);
    conv_ = stack_rows({pad_matrix(need(t, "q_conv.weight"), qk_, taps_), pad_matrix(need(t, "k_conv.weight"), qk_, taps_),
                        pad_matrix(need(t, "v_conv.weight"), v_, taps_)});
    (void)qk; (void)v;
    A_log_ = need(t, "A_log");
    dt_bias_ = need(t, "dt_bias");
    out_norm_ = need(t, "out_norm.weight");
    w_o_ = pad_matrix(need(t, "o_proj.weight"), hidden_, v_);      // the read-out's width as whole 16-byte vectors
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {state_floats() + (int64_t)(taps_ - 1) * channels_};
    n.state_dtype = DType::F32;
    return n;
  }
  // Which sequence of the step every token belongs to.
  const char* step_inputs_key() const override { return "delta.token_seq"; }
  void step_inputs(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) override { token_sequences(step, out); }

  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::State) throw EngineError("the delta rule was handed a cache entry without state");
    Kernels& k = kernels;
    const Tensor proj = k.gemm(x, w_in_);
    const Tensor a = k.gemm_columns(proj, decay_col_, w_decay_up_);
    const Tensor gate = k.gemm_columns(proj, gate_col_, w_gate_up_);
    Tensor qkv = k.delta_conv(proj, conv_, cache.state, state_floats(), ctx.inputs.at("delta.token_seq"), ctx.cu_q, ctx.positions, ctx.state_slots);
    const Tensor decay = k.delta_prep(qkv, 0, qk_, G_, H_, d_, unit_eps_, 1.f / std::sqrt((float)d_), a, dt_bias_, A_log_);
    const Tensor o = k.delta_rule(qkv, 0, (int)qk_, (int)(2 * qk_), decay, proj, beta_col_, cache.state, ctx.cu_q, ctx.positions, ctx.state_slots,
                                  H_, G_, d_, dv_);
    return k.gemm(k.delta_out(o, gate, out_norm_, H_, dv_, eps_, v_), w_o_);
  }

 private:
  int64_t state_floats() const { return (int64_t)H_ * d_ * dv_; }
  int64_t hidden_;
  int H_, G_, d_, dv_, taps_;
  int64_t decay_rank_, gate_rank_;
  float eps_, unit_eps_;
  int64_t qk_ = 0, v_ = 0, channels_ = 0, beta_col_ = 0, decay_col_ = 0, gate_col_ = 0;
  Tensor w_in_, w_decay_up_, w_gate_up_, conv_, A_log_, dt_bias_, out_norm_, w_o_;
};

// Gated linear attention with one decay per head and key channel.  For the mixer's input h:
//   q = W_q h * key size^(-1/2), k = W_k h (heads x key size), v = W_v h (heads x value size);
//   g = sigmoid(W_a2 (W_a1 h) + b_a2)^(1 / decay_root) per head and key channel;
//   per head, token by token:  S <- diag(g) S + k v^T;  o = S^T q;
//   y = o / sqrt(mean(o^2) + eps) * w_norm * silu(W_g h) per head; out = W_o y.
// A request's state slot holds the heads' S in 32-bit, zero at the request's start.  The five input projections are one
// launch (their weights stacked, each section padded to a multiple of 8 rows with zero rows, so that the decay's second
// projection reads its columns in place); decays, recurrence and read-out are kernels of delta.hip, all in 32-bit: the
// recurrence is the delta rule's walk without its correction term.
class GatedLinearAttention : public Mixer {
 public:
  GatedLinearAttention(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), H_((int)s.integer("num_heads")), d_((int)s.integer("key_dim")), dv_((int)s.integer("value_dim")),
        decay_rank_(s.integer("decay_rank", 0)), root_((float)s.number("decay_root", 1.0)), eps_((float)s.number("eps")) {
    if (H_ < 1 || d_ < 1 || dv_ < 1 || d_ > 1024) throw ConfigError("linear attention: heads of " + std::to_string(d_) + " x " + std::to_string(dv_));
    if (!(root_ > 0.f)) throw ConfigError("linear attention: 'decay_root' must be positive");
    qk_ = round_up((int64_t)H_ * d_, 8);
    v_ = round_up((int64_t)H_ * dv_, 8);
  }
  std::vector<ParamDecl> params() const override {
    const int64_t hd = (int64_t)H_ * d_, hv = (int64_t)H_ * dv_;
    const int64_t ra = decay_rank_ > 0 ? decay_rank_ : -1;      // 0: the rank is whatever the stored tensors have
    ParamDecl q{"q_proj.weight", {hd, hidden_}}, kk{"k_proj.weight", {hd, hidden_}}, vv{"v_proj.weight", {hv, hidden_}};
    q.p0 = kk.p0 = vv.p0 = 0.1;
    ParamDecl a1{"decay_down.weight", {ra, hidden_}}, a2{"decay_up.weight", {hd, ra}};
    a1.free_size = a2.free_size = std::max<int64_t>(8, hidden_ / 16);
    a2.p0 = 0.5;
    ParamDecl bias{"decay_up.bias", {hd}, true, true, 1.0, 5.0}, norm{"out_norm.weight", {(int64_t)dv_}, true, true, 0.9, 1.1};
    return {q, kk, vv, {"gate_proj.weight", {hv, hidden_}}, a1, a2, bias, norm, {"o_proj.weight", {hidden_, hv}}};
  }
  void load(std::map<std::string, Tensor>& t) override {
    const Tensor a1 = need(t, "decay_down.weight"), a2 = need(t, "decay_up.weight");
    if (a1.dim(0) != a2.dim(1)) throw EngineError("linear attention: the decay's two projections do not fit each other: " + a1.describe() + " with " + a2.describe());
    const int64_t ra = round_up(a1.dim(0), 8);
    w_in_ = stack_rows({pad_matrix(need(t, "q_proj.weight"), qk_, hidden_), pad_matrix(need(t, "k_proj.weight"), qk_, hidden_),
                        pad_matrix(need(t, "v_proj.weight"), v_, hidden_), pad_matrix(need(t, "gate_proj.weight"), v_, hidden_),
                        pad_matrix(a1, ra, hidden_)});
    gate_col_ = 2 * qk_ + v_;
    decay_col_ = gate_col_ + v_;
    w_decay_up_ = pad_matrix(a2, a2.dim(0), ra);
    decay_bias_ = need(t, "decay_up.bias");
    out_norm_ = need(t, "out_norm.weight");
    w_o_ = pad_matrix(need(t, "o_proj.weight"), hidden_, v_);      // the read-out's width as whole 16-byte vectors
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {(int64_t)H_ * d_ * dv_};
    n.state_dtype = DType::F32;
    return n;
  }
  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::State) throw EngineError("linear attention was handed a cache entry without state");
    Kernels& k = kernels;
    const Tensor proj = k.gemm(x, w_in_);
    const Tensor decay = k.gla_decay(k.gemm_columns(proj, decay_col_, w_decay_up_), decay_bias_, H_, d_, root_);
    const Tensor o = k.gla_rule(proj, 0, qk_, 2 * qk_, decay, cache.state, ctx.cu_q, ctx.positions, ctx.state_slots, H_, d_, dv_,
                                1.f / std::sqrt((float)d_));
    return k.gemm(k.gated_head_norm(o, proj, gate_col_, out_norm_, H_, dv_, eps_, 1, v_), w_o_);
  }

 private:
  int64_t hidden_;
  int H_, d_, dv_;
  int64_t decay_rank_;
  float root_, eps_;
  int64_t qk_ = 0, v_ = 0, gate_col_ = 0, decay_col_ = 0;
  Tensor w_in_, w_decay_up_, decay_bias_, out_norm_, w_o_;
};

// A layer without a feed-forward names this kind; an arrangement that allows it never calls it.
class NoFeedForward : public FeedForward {
 public:
  NoFeedForward(const PartSpec&, Kernels& k) : FeedForward(k) {}
  Tensor forward(const Tensor&, StepContext&) override { throw EngineError("a layer without a feed-forward was asked to run one"); }
};

// A residual stream x in 32-bit, a norm before and after each sublayer, and (kind "sandwich_depth"; kind "sandwich" ends
// after the two sublayers, and needs the numbers residual_mult and hidden_size alone) a weighted sum over the stream's earlier
// states at the layer's end:
//   x <- x + m * norm_mixer_out(mixer(norm_mixer_in(x)));  x <- x + m * norm_ffn_out(ffn(norm_ffn_in(x))) (if the
//   layer has a feed-forward);  X_(i+1) = x;  passed on: sum over j <= i + 1 of depth_weights[j] * X_j,
// where X_0 is what the embedding gave and i = `depth`, the layer's place in the run order.  The states of a step lie
// in one tensor [states, tokens, width] that the first layer of the step takes from the arena (ctx.carry).
class SandwichDepthBlock : public Block {
 public:
  SandwichDepthBlock(Kernels& k, std::unique_ptr<Mixer> mixer, std::unique_ptr<FeedForward> ffn, std::map<std::string, std::unique_ptr<Norm>> norms,
                     const std::map<std::string, double>& numbers)
      : Block(k), mixer_(std::move(mixer)), ffn_(std::move(ffn)), norms_(std::move(norms)) {
    auto number = [&](const char* name) {
      auto it = numbers.find(name);
      if (it == numbers.end()) throw ConfigError(std::string("a sandwich_depth block needs the number '") + name + "'");
      return it->second;
    };
    mult_ = (float)number("residual_mult");
    deep_ = numbers.count("states") > 0;
    depth_ = deep_ ? (int)number("depth") : 0;
    states_ = deep_ ? (int)number("states") : 2;
    hidden_ = (int64_t)number("hidden_size");
    if (depth_ < 0 || depth_ + 1 >= states_) throw ConfigError("a sandwich_depth block at depth " + std::to_string(depth_) + " of " + std::to_string(states_) + " states");
    has_ffn_ = dynamic_cast<NoFeedForward*>(ffn_.get()) == nullptr;
    for (const char* n : {"mixer_in", "mixer_out"})
      if (!norms_.count(n)) throw ConfigError(std::string("a sandwich_depth block needs the norms 'mixer_in' and 'mixer_out'; missing: ") + n);
    if (has_ffn_ && (!norms_.count("ffn_in") || !norms_.count("ffn_out")))
      throw ConfigError("a sandwich_depth block with a feed-forward needs the norms 'ffn_in' and 'ffn_out'");
  }
  std::vector<ParamDecl> params() const override {
    if (!deep_) return {};
    ParamDecl w{"depth_weights", {(int64_t)depth_ + 2}, true, true, 0.0, 2.0 / (depth_ + 2)};
    return {w};
  }
  void load(std::map<std::string, Tensor>& t) override {
    if (deep_) weights_ = need(t, "depth_weights");
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c = {{"mixer", mixer_.get()}, {"feed_forward", ffn_.get()}};
    for (auto& n : norms_) c.emplace_back("norms." + n.first, n.second.get());
    return c;
  }
  Mixer& mixer() override { return *mixer_; }
  std::pair<Tensor, Tensor> forward(const Tensor& hidden, Tensor residual, StepContext& ctx, CacheEntry& cache) override {
    Kernels& k = kernels;
    if (hidden.dtype != DType::F32 || hidden.shape.size() != 2 || hidden.dim(1) != hidden_)
      throw EngineError("a sandwich_depth block takes the 32-bit residual stream, not " + hidden.describe());
    const int64_t T = hidden.dim(0);
    if (!deep_) {
      // The plain arrangement (kind "sandwich"): the stream itself is passed on.
      Tensor stream = hidden;
      const Tensor mixed = mixer_->forward(norms_["mixer_in"]->forward(hidden), ctx, cache);
      norms_["mixer_out"]->forward_scaled_add(mixed, hidden, stream, mult_);
      if (has_ffn_) {
        const Tensor fed = ffn_->forward(norms_["ffn_in"]->forward(stream), ctx);
        norms_["ffn_out"]->forward_scaled_add(fed, stream, stream, mult_);
      }
      return {stream, residual};
    }
    Tensor& states = ctx.carry["stream.states"];
    if (depth_ == 0) {
      states = k.empty({(int64_t)states_, T, hidden_}, DType::F32);
      hip_check(hipMemcpyAsync(states.data, hidden.data, hidden.bytes(), hipMemcpyDeviceToDevice, k.stream), "keeping the embedding's output");
    }
    if (!states.data || states.dim(0) != states_ || states.dim(1) != T) throw EngineError("a sandwich_depth block found no states of this step's stream");
    Tensor result = states.rows(depth_ + 1, 1).view({T, hidden_});
    const Tensor mixed = mixer_->forward(norms_["mixer_in"]->forward(hidden), ctx, cache);
    if (has_ffn_) {
      Tensor mid = k.empty({T, hidden_}, DType::F32);
      norms_["mixer_out"]->forward_scaled_add(mixed, hidden, mid, mult_);
      const Tensor fed = ffn_->forward(norms_["ffn_in"]->forward(mid), ctx);
      norms_["ffn_out"]->forward_scaled_add(fed, mid, result, mult_);
    } else {
      norms_["mixer_out"]->forward_scaled_add(mixed, hidden, result, mult_);
    }
    return {k.stream_mix(states, weights_, depth_ + 2), residual};
  }

 private:
  std::unique_ptr<Mixer> mixer_;
  std::unique_ptr<FeedForward> ffn_;
  std::map<std::string, std::unique_ptr<Norm>> norms_;
  float mult_ = 1.f;
  int depth_ = 0, states_ = 0;
  int64_t hidden_ = 0;
  bool has_ffn_ = true, deep_ = true;    // deep_: the weighted sum over earlier states ends the layer
  Tensor weights_;
};

// A state-space recurrence with one decay per head.  For the mixer's input h, with inner = heads * value size P, the
// state size N and G groups:  W_in h = [z: inner | x: inner | B: G N | C: G N | dt: heads];  x, B and C together pass a
// short causal convolution per channel (taps [channels, K] with the last tap the current token's, a bias, zeros before a
// sequence's start) and silu;  dt <- softplus(dt + dt_bias);  per head (its B and C are those of group head / (heads /
// G)), token by token:  S <- exp(-exp(A_log) dt) S + dt B x^T  (S is N x P),  y = S^T C + D x;  the heads' y side by
// side times silu(z), divided in `norm_groups` equal parts each by its own root mean square, times a weight; then W_o.
// A request's state slot holds the heads' S in 32-bit and the convolution's last K - 1 inputs.  Everything between the
// two projections is 32-bit (ssm.hip and the convolution of delta.hip).
class StateSpace : public Mixer {
 public:
  StateSpace(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), H_((int)s.integer("num_heads")), P_((int)s.integer("value_dim")),
        N_((int)s.integer("state_dim")), G_((int)s.integer("groups")), parts_((int)s.integer("norm_groups", 1)),
        taps_((int)s.integer("conv_taps")), eps_((float)s.number("eps")) {
    if (H_ % G_) throw ConfigError(std::to_string(H_) + " heads are not a multiple of " + std::to_string(G_) + " groups");
    if (taps_ < 1 || taps_ > 17) throw ConfigError("a short convolution of " + std::to_string(taps_) + " taps: 1 to 17 are built");
    if (N_ > 256) throw ConfigError("a state of " + std::to_string(N_) + " rows a head: up to 256 are built");
    inner_ = (int64_t)H_ * P_;
    if (parts_ < 1 || inner_ % parts_) throw ConfigError(std::to_string(parts_) + " norm groups do not divide " + std::to_string(inner_) + " channels");
    channels_ = inner_ + 2 * (int64_t)G_ * N_;
  }
  std::vector<ParamDecl> params() const override {
    auto uniform = [](const char* name, std::vector<int64_t> shape, double lo, double hi) {
      ParamDecl p{name, std::move(shape), true, true, lo, hi};
      return p;
    };
    ParamDecl in{"in_proj.weight", {inner_ + channels_ + H_, hidden_}}, taps{"conv.weight", {channels_, taps_}};
    in.p0 = 0.05;
    taps.p0 = 0.3;
    return {in, taps, uniform("conv.bias", {channels_}, -0.1, 0.1), uniform("dt_bias", {(int64_t)H_}, -2.0, 0.0), uniform("A_log", {(int64_t)H_}, -1.0, 1.0),
            uniform("D", {(int64_t)H_}, 0.5, 1.5), uniform("out_norm.weight", {inner_}, 0.9, 1.1), {"o_proj.weight", {hidden_, inner_}}};
  }
  void load(std::map<std::string, Tensor>& t) override {
    w_in_ = need(t, "in_proj.weight");
    conv_ = need(t, "conv.weight");
    conv_bias_ = need(t, "conv.bias");
    if (conv_bias_.dtype != kernels.dtype()) throw EngineError("the convolution's bias must have the element type");
    dt_bias_ = need(t, "dt_bias");
    A_log_ = need(t, "A_log");
    D_ = need(t, "D");
    out_norm_ = need(t, "out_norm.weight");
    inner_run_ = round_up(inner_, 8);                              // the read-out's width as whole 16-byte vectors
    w_o_ = pad_matrix(need(t, "o_proj.weight"), hidden_, inner_run_);
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {state_floats() + (int64_t)(taps_ - 1) * channels_};
    n.state_dtype = DType::F32;
    return n;
  }
  const char* step_inputs_key() const override { return "delta.token_seq"; }
  void step_inputs(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) override { token_sequences(step, out); }

  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::State) throw EngineError("the state-space mixer was handed a cache entry without state");
    Kernels& k = kernels;
    const Tensor proj = k.gemm(x, w_in_);
    const Tensor xbc = k.delta_conv(proj, conv_, cache.state, state_floats(), ctx.inputs.at("delta.token_seq"), ctx.cu_q, ctx.positions,
                                    ctx.state_slots, inner_, &conv_bias_);
    const Tensor y = k.ssm_scan(xbc, inner_, inner_ + (int64_t)G_ * N_, proj, inner_ + channels_, dt_bias_, A_log_, D_, cache.state, ctx.cu_q,
                                ctx.positions, ctx.state_slots, H_, G_, N_, P_);
    return k.gemm(k.ssm_gate_norm(y, proj, 0, out_norm_, parts_, eps_, inner_run_), w_o_);
  }

 private:
  int64_t state_floats() const { return (int64_t)H_ * P_ * N_; }
  int64_t hidden_;
  int H_, P_, N_, G_, parts_, taps_;
  float eps_;
  int64_t inner_ = 0, channels_ = 0, inner_run_ = 0;
  Tensor w_in_, conv_, conv_bias_, dt_bias_, A_log_, D_, out_norm_, w_o_;
};

// Two mixers side by side that read the same input: out = (norm(left(h)) * w_left + norm(right(h)) * w_right) / 2, each
// output divided by its root mean square over the width, in 32-bit.  One of them may keep pages and the other a state:
// the pair asks for both, and each half gets its own.
class PairMean : public Mixer {
 public:
  PairMean(const PartSpec& s, Kernels& k) : Mixer(k), hidden_(s.integer("hidden_size")), eps_((float)s.number("eps")) {
    const PartSpec *l = s.part("left_mixer"), *r = s.part("right_mixer");
    if (!l || !r) throw ConfigError("a pair of mixers needs the parts 'left_mixer' and 'right_mixer'");
    left_ = build_part<Mixer>("mixer", *l, k);
    right_ = build_part<Mixer>("mixer", *r, k);
    const CacheNeed a = left_->cache_need(), b = right_->cache_need();
    if ((a.kind == CacheNeed::Pages && b.kind == CacheNeed::Pages) || (a.kind == CacheNeed::State && b.kind == CacheNeed::State))
      throw ConfigError("a pair of mixers that both keep pages, or both a state, is not built");
  }
  std::vector<ParamDecl> params() const override {
    ParamDecl l{"left_out", {hidden_}, true, true, 0.9, 1.1}, r{"right_out", {hidden_}, true, true, 0.9, 1.1};
    return {l, r};
  }
  std::vector<std::pair<std::string, Part*>> children() override { return {{"left", left_.get()}, {"right", right_.get()}}; }
  void load(std::map<std::string, Tensor>& t) override {
    w_left_ = need(t, "left_out");
    w_right_ = need(t, "right_out");
  }
  CacheNeed cache_need() const override {
    const CacheNeed a = left_->cache_need(), b = right_->cache_need();
    CacheNeed n = a.kind == CacheNeed::Pages ? a : (b.kind == CacheNeed::Pages ? b : (a.kind == CacheNeed::State ? a : b));
    const CacheNeed& other = a.kind == CacheNeed::State ? a : b;
    if (n.kind == CacheNeed::Pages && other.kind == CacheNeed::State) {
      n.state_shape = other.state_shape;
      n.state_dtype = other.state_dtype;
    }
    return n;
  }
  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    const Tensor l = half(*left_, x, ctx, cache), r = half(*right_, x, ctx, cache);
    return kernels.stream_pair_norm(l, w_left_, r, w_right_, eps_, 0.5f, 0.5f);
  }

 private:
  // A half sees the entry as the kind it asked for.
  Tensor half(Mixer& m, const Tensor& x, StepContext& ctx, CacheEntry& cache) {
    const CacheNeed::Kind kind = m.cache_need().kind;
    if (kind == cache.kind) return m.forward(x, ctx, cache);
    CacheEntry own = cache;
    own.kind = kind;
    if (kind == CacheNeed::State && !own.state.data) throw EngineError("a pair of mixers was handed a cache entry without the state of one half");
    return m.forward(x, ctx, own);
  }
  int64_t hidden_;
  float eps_;
  std::unique_ptr<Mixer> left_, right_;
  Tensor w_left_, w_right_;
};

// A mixture of `experts` small feed-forward layers without biases, W_down max(W_up h, 0)^2, of which every token uses
// `top`: router logits W_router h in 32-bit, a softmax over all experts, the `top` largest scores, divided by their
// sum plus weight_eps; the output is the weighted sum of the chosen experts' outputs, in 32-bit.  The experts' weights
// lie stacked, [experts, ff, width] and [experts, width, ff] (ff padded to a multiple of 64 with zeros), and the two
// projections run as grouped products over the (token, choice) pairs sorted by expert (moe.hip, gemm.hip).
//
// Further numbers, all optional: router_bias (a bias per expert on the logits, which choice and weights both see; with
// weight_eps 0 the weights are then the softmax over the chosen logits alone), gated (an expert is
// W_down (g * sigmoid(glu_slope * g) * (u + up_shift)) with g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit)),
// shared_size (> 0: one more expert of that inner size and the same form, with shared_limit, that every token uses
// with weight 1; its output is added to the sum), score (1: the weights are the logistic function of the chosen logits, not
// divided by anything), weigh_input (1: the output is the sum of expert(weight * h); since W (w h) = w (W h), the weight
// multiplies the gate and up outputs before their clamps, and the sum adds the experts' outputs as they are).
class RoutedExperts : public FeedForward {
 public:
  RoutedExperts(const PartSpec& s, Kernels& k)
      : FeedForward(k), hidden_(s.integer("hidden_size")), inter_(s.integer("intermediate_size")), experts_((int)s.integer("experts")),
        top_((int)s.integer("top")), weight_eps_((float)s.number("weight_eps", 0.0)), bias_(s.integer("router_bias", 0) != 0),
        gated_(s.integer("gated", 0) != 0), limit_((float)s.number("limit", 0.0)), slope_((float)s.number("glu_slope", 1.0)),
        shift_((float)s.number("up_shift", 0.0)), shared_(s.integer("shared_size", 0)), shared_limit_((float)s.number("shared_limit", 0.0)),
        score_((int)s.integer("score", 0)), weigh_input_(s.integer("weigh_input", 0) != 0) {
    if (score_ < 0 || score_ > 1) throw ConfigError("experts: 'score' is 0 (softmax) or 1 (the logistic function of a chosen logit)");
    if (weigh_input_ && (!gated_ || shared_ > 0)) throw ConfigError("experts whose weights scale their inputs are built in the gated form, without a shared expert");
    if (experts_ < 1 || top_ < 1 || top_ > experts_) throw ConfigError("a mixture of " + std::to_string(experts_) + " experts cannot choose " + std::to_string(top_));
    if (gated_ && !(limit_ > 0.f)) throw ConfigError("gated experts need a positive 'limit'");
    if (shared_ < 0 || (shared_ > 0 && (!gated_ || !(shared_limit_ > 0.f))))
      throw ConfigError("a shared expert is built in the gated form, with a positive 'shared_limit'");
  }
  std::vector<ParamDecl> params() const override {
    std::vector<ParamDecl> p = {{"router.weight", {(int64_t)experts_, hidden_}}};
    p[0].p0 = 0.1;
    if (bias_) {
      ParamDecl b{"router.bias", {(int64_t)experts_}, true, true, -0.5, 0.5};
      p.push_back(b);
    }
    for (int e = 0; e < experts_; ++e) {
      if (gated_) p.push_back({"experts." + std::to_string(e) + ".gate_proj.weight", {inter_, hidden_}});
      p.push_back({"experts." + std::to_string(e) + ".up_proj.weight", {inter_, hidden_}});
      p.push_back({"experts." + std::to_string(e) + ".down_proj.weight", {hidden_, inter_}});
    }
    if (shared_ > 0) {
      p.push_back({"shared.gate_proj.weight", {shared_, hidden_}});
      p.push_back({"shared.up_proj.weight", {shared_, hidden_}});
      p.push_back({"shared.down_proj.weight", {hidden_, shared_}});
    }
    return p;
  }
  void load(std::map<std::string, Tensor>& t) override {
    router_ = need(t, "router.weight");
    const int64_t padded = round_up(inter_, 64);              // whole pairs of slabs, so that the tile product takes it
    std::vector<Tensor> up, down;
    if (bias_) router_bias_ = need(t, "router.bias");
    if (shared_ > 0) {
      const int64_t sp = round_up(shared_, 64);
      w_shared_in_ = stack_rows({pad_matrix(need(t, "shared.gate_proj.weight"), sp, hidden_), pad_matrix(need(t, "shared.up_proj.weight"), sp, hidden_)});
      w_shared_down_ = pad_matrix(need(t, "shared.down_proj.weight"), hidden_, sp);
    }
    for (int e = 0; e < experts_; ++e) {
      // A gated expert's first product gives the gate's outputs and then the up projection's, each padded alike.
      if (gated_) up.push_back(pad_matrix(need(t, "experts." + std::to_string(e) + ".gate_proj.weight"), padded, hidden_));
      up.push_back(pad_matrix(need(t, "experts." + std::to_string(e) + ".up_proj.weight"), padded, hidden_));
      Tensor d = pad_matrix(need(t, "experts." + std::to_string(e) + ".down_proj.weight"), hidden_, padded);
      down.push_back(d.view({hidden_ * padded / 8, 8}));     // stacked as rows of one width whatever the matrices' own
    }
    w_up_ = stack_rows(up).view({(int64_t)experts_, (gated_ ? 2 : 1) * padded, hidden_});
    w_down_ = stack_rows(down).view({(int64_t)experts_, hidden_, padded});
  }
  Tensor forward(const Tensor& x, StepContext&) override {
    Kernels& k = kernels;
    const int64_t pairs = x.dim(0) * top_;
    const Tensor* bias = bias_ ? &router_bias_ : nullptr;
    Tensor shared;
    if (shared_ > 0) shared = k.gemm(k.moe_glu(k.gemm(x, w_shared_in_), shared_limit_, slope_, shift_), w_shared_down_);
    const Tensor* extra = shared_ > 0 ? &shared : nullptr;
    // Few rows an expert: products over tiles of 16 rows that stream an expert's weights once a tile.  Many (prompts):
    // the rows are sorted by expert into blocks of 128 and go through the engine's tile product, every block with its
    // expert's matrix.  Both are launched from numbers on the GPU alone and give the same bits.
    if (pairs < (int64_t)kRowsAnExpertForTiles * experts_ || !k.gemm_grouped_takes(hidden_) || !k.gemm_grouped_takes(w_down_.dim(2))) {
      const Kernels::MoePlan plan = k.moe_route_scored(x, router_, top_, weight_eps_, 16, bias, score_);
      if (weigh_input_)
        return k.moe_sum_unweighed(k.moe_down(k.moe_glu_weighed(k.moe_up_plain(x, w_up_, plan), limit_, slope_, shift_, plan), w_down_, plan), plan);
      const Tensor act = gated_ ? k.moe_glu(k.moe_up_plain(x, w_up_, plan), limit_, slope_, shift_) : k.moe_up(x, w_up_, plan);
      return k.moe_sum(k.moe_down(act, w_down_, plan), plan, extra);
    }
    const Kernels::MoePlan plan = k.moe_route_scored(x, router_, top_, weight_eps_, 128, bias, score_);
    Tensor act = k.gemm_grouped(k.gather_rows(x, plan.row_token), w_up_, plan.tile_expert);
    if (weigh_input_) return k.moe_sum_unweighed(k.gemm_grouped(k.moe_glu_weighed(act, limit_, slope_, shift_, plan), w_down_, plan.tile_expert), plan);
    if (gated_) act = k.moe_glu(act, limit_, slope_, shift_);
    else k.relu_square(act);
    return k.moe_sum(k.gemm_grouped(act, w_down_, plan.tile_expert), plan, extra);
  }
  static constexpr int kRowsAnExpertForTiles = 32;

 private:
  int64_t hidden_, inter_;
  int experts_, top_;
  float weight_eps_;
  bool bias_, gated_;
  float limit_, slope_, shift_;
  int64_t shared_;
  float shared_limit_;
  int score_;              // 0: softmax scores; 1: a chosen expert's weight is the logistic function of its logit
  bool weigh_input_;       // a weight scales what its expert reads (the gate and up outputs before their clamps), not what it gives
  Tensor router_, router_bias_, w_up_, w_down_, w_shared_in_, w_shared_down_;
};

// Mixer and feed-forward side by side on a residual stream x in 32-bit: x <- x + (mixer(norm_mixer_in(x)) +
// ffn(norm_ffn_in(x))), both norms of the same x; without a feed-forward, x <- x + mixer(norm_mixer_in(x)).
class ParallelSumBlock : public Block {
 public:
  ParallelSumBlock(Kernels& k, std::unique_ptr<Mixer> mixer, std::unique_ptr<FeedForward> ffn, std::map<std::string, std::unique_ptr<Norm>> norms,
                   const std::map<std::string, double>& numbers)
      : Block(k), mixer_(std::move(mixer)), ffn_(std::move(ffn)), norms_(std::move(norms)) {
    auto it = numbers.find("hidden_size");
    if (it == numbers.end()) throw ConfigError("a parallel_sum block needs the number 'hidden_size'");
    hidden_ = (int64_t)it->second;
    has_ffn_ = dynamic_cast<NoFeedForward*>(ffn_.get()) == nullptr;
    if (!norms_.count("mixer_in")) throw ConfigError("a parallel_sum block needs the norm 'mixer_in'");
    if (has_ffn_ && !norms_.count("ffn_in")) throw ConfigError("a parallel_sum block with a feed-forward needs the norm 'ffn_in'");
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c = {{"mixer", mixer_.get()}, {"feed_forward", ffn_.get()}};
    for (auto& n : norms_) c.emplace_back("norms." + n.first, n.second.get());
    return c;
  }
  Mixer& mixer() override { return *mixer_; }
  std::pair<Tensor, Tensor> forward(const Tensor& hidden, Tensor residual, StepContext& ctx, CacheEntry& cache) override {
    if (hidden.dtype != DType::F32 || hidden.shape.size() != 2 || hidden.dim(1) != hidden_)
      throw EngineError("a parallel_sum block takes the 32-bit residual stream, not " + hidden.describe());
    Tensor stream = hidden;
    const Tensor mixed = mixer_->forward(norms_["mixer_in"]->forward(hidden), ctx, cache);
    if (has_ffn_) {
      const Tensor fed = ffn_->forward(norms_["ffn_in"]->forward(hidden), ctx);
      kernels.stream_add(stream, mixed, &fed);
    } else {
      kernels.stream_add(stream, mixed, nullptr);
    }
    return {stream, residual};
  }

 private:
  std::unique_ptr<Mixer> mixer_;
  std::unique_ptr<FeedForward> ffn_;
  std::map<std::string, std::unique_ptr<Norm>> norms_;
  int64_t hidden_ = 0;
  bool has_ffn_ = true;
};

// A weight laid out anew on the host: element (i, j) of the result [rows, cols] is the source's element from(i, j), or zero
// where that gives a negative row.  For arrangements that a strided copy cannot express (a transpose a head, say).
Tensor rearranged(const Tensor& w, int64_t rows, int64_t cols, const std::function<std::pair<int64_t, int64_t>(int64_t, int64_t)>& from) {
  if (w.shape.size() != 2) throw EngineError("a weight of " + w.describe() + " cannot be rearranged as a matrix");
  const size_t e = (size_t)dtype_bytes(w.dtype);
  std::vector<char> src(w.bytes()), dst((size_t)(rows * cols) * e, 0);
  if (w.numel()) hip_check(hipMemcpy(src.data(), w.data, w.bytes(), hipMemcpyDeviceToHost), "reading a weight back");
  for (int64_t i = 0; i < rows; ++i)
    for (int64_t j = 0; j < cols; ++j) {
      const auto ij = from(i, j);
      if (ij.first < 0) continue;
      if (ij.first >= w.dim(0) || ij.second < 0 || ij.second >= w.dim(1)) throw EngineError("a weight's rearrangement reads outside " + w.describe());
      std::copy_n(src.data() + (size_t)(ij.first * w.dim(1) + ij.second) * e, e, dst.data() + (size_t)(i * cols + j) * e);
    }
  Tensor out = zero_weight({rows, cols}, w.dtype);
  if (out.numel()) hip_check(hipMemcpy(out.data, dst.data(), dst.size(), hipMemcpyHostToDevice), "writing a weight");
  return out;
}

// Attention through a latent.  For the mixer's input h, with H heads, per head d entries that are not rotated and dr that
// are, value size dv, latent size r and query latent size rq:
//   c_q = norm(W_dq h) (weight dq.norm), q = W_uq c_q, head by head [d | dr];  W_dkv h = [latent: r | key part: dr];
//   c = norm(latent) (weight dkv.norm); the key part is rotated by the position and serves every head;
//   head j: k_j = W_uk[j] c, v_j = W_uv[j] c; score = (q_flat . k_j + rotate(q_rot) . rotated key part) * scale;
//   softmax over the keys so far; the heads side by side times sigmoid(W_g h); then W_o.
// Only c and the rotated key part are kept: the cache has one kv head whose key row is [c | rotated part | 0] and whose
// value row is [c | 0], D = r + dr rounded up to 16 entries.  Since q_flat . (W_uk[j] c) = (W_uk[j]^T q_flat) . c, head j's
// query meets the cache as [W_uk[j]^T q_flat | rotate(q_rot) | 0], and its output is W_uv[j] times the weighted sum of the
// cached c: two products a head (gemm_heads) around the engine's paged attention kernels, whose weights are 32-bit.
// own_kv 0: the layer has no W_dkv and reads the cache of an earlier layer of the same latent and rotation, with W_uk,
// W_uv, queries and everything else of its own.  Sizes that are no whole 16-byte vectors are padded with zeros in the
// weights at load.
class LatentAttention : public Mixer {
 public:
  LatentAttention(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), H_((int)s.integer("num_heads")), d_((int)s.integer("head_dim")), dr_((int)s.integer("rotary_dim")),
        dv_((int)s.integer("value_dim")), r_((int)s.integer("kv_rank")), rq_((int)s.integer("q_rank")), scale_((float)s.number("scale")),
        eps_((float)s.number("eps")), own_kv_(s.integer("own_kv", 1) != 0), gate_(s.integer("output_gate", 0) != 0) {
    D_ = (int)round_up((int64_t)r_ + dr_, 16);
    if (H_ < 1 || d_ < 1 || dr_ < 2 || dr_ % 2 || dv_ < 1 || r_ < 1 || rq_ < 1) throw ConfigError("latent attention: bad sizes");
    if (D_ > 256) throw ConfigError("latent attention: a latent of " + std::to_string(r_) + " with " + std::to_string(dr_) + " rotated entries: the attention kernels take up to 256 together");
    const PartSpec* p = s.part("position");
    if (!p) throw ConfigError("latent attention needs the part 'position'");
    position_ = build_part<PositionEncoding>("position", *p, k);
    dp_ = round_up(d_, 8);
    qs_ = dp_ + round_up(dr_, 8);
    rqp_ = round_up(rq_, 8);
    kvp_ = round_up((int64_t)r_ + dr_, 8);
    dvp_ = round_up(dv_, 8);
  }
  std::vector<ParamDecl> params() const override {
    ParamDecl qn{"q_down_norm.weight", {(int64_t)rq_}, true, true, 0.9, 1.1}, kn{"kv_down_norm.weight", {(int64_t)r_}, true, true, 0.9, 1.1};
    ParamDecl uq{"q_up.weight", {(int64_t)H_ * (d_ + dr_), (int64_t)rq_}}, uk{"k_up.weight", {(int64_t)H_ * d_, (int64_t)r_}},
        uv{"v_up.weight", {(int64_t)H_ * dv_, (int64_t)r_}};
    uq.p0 = uk.p0 = uv.p0 = 0.06;
    std::vector<ParamDecl> p = {{"q_down.weight", {(int64_t)rq_, hidden_}}, qn, uq, uk, uv, {"o_proj.weight", {hidden_, (int64_t)H_ * dv_}}};
    if (own_kv_) {
      p.push_back({"kv_down.weight", {(int64_t)r_ + dr_, hidden_}});
      p.push_back(kn);
    }
    if (gate_) p.push_back({"gate_proj.weight", {(int64_t)H_ * dv_, hidden_}});
    return p;
  }
  std::vector<std::pair<std::string, Part*>> children() override { return {{"position", position_.get()}}; }
  void load(std::map<std::string, Tensor>& t) override {
    if (!position_->angle_frequencies()) throw ConfigError("latent attention is built for rotations by computed angles");
    // One launch projects the query's latent, the latent with its key part (where the layer has them) and the gate.
    std::vector<Tensor> rows = {pad_matrix(need(t, "q_down.weight"), rqp_, hidden_)};
    if (own_kv_) rows.push_back(pad_matrix(need(t, "kv_down.weight"), kvp_, hidden_));
    if (gate_) rows.push_back(pad_row_blocks(need(t, "gate_proj.weight"), H_, dv_, dvp_));
    w_in_ = rows.size() > 1 ? stack_rows(rows) : rows[0];
    kv_col_ = own_kv_ ? rqp_ : -1;
    gate_col_ = rqp_ + (own_kv_ ? kvp_ : 0);
    q_norm_ = need(t, "q_down_norm.weight");
    if (own_kv_) kv_norm_ = need(t, "kv_down_norm.weight");
    const int64_t d = d_, dr = dr_, dp = dp_, qs = qs_, r = r_, dv = dv_, D = D_;
    // A head's query rows as [d | zeros to dp | dr | zeros to qs], the columns padded to the padded latent.
    w_uq_ = rearranged(need(t, "q_up.weight"), (int64_t)H_ * qs, rqp_, [=](int64_t i, int64_t j) -> std::pair<int64_t, int64_t> {
      const int64_t h = i / qs, e = i % qs;
      if (j >= rq_) return {-1, 0};
      if (e < d) return {h * (d + dr) + e, j};
      if (e >= dp && e < dp + dr) return {h * (d + dr) + d + (e - dp), j};
      return {-1, 0};
    });
    // Head h's W_uk transposed: [r, dp], so that a product a head takes q_flat to the latent's side.
    w_absorb_ = rearranged(need(t, "k_up.weight"), (int64_t)H_ * r, dp, [=](int64_t i, int64_t j) -> std::pair<int64_t, int64_t> {
                  if (j >= d) return {-1, 0};
                  return {(i / r) * d + j, i % r};
                }).view({(int64_t)H_, r, dp});
    // Head h's W_uv over a whole cache row: [dvp, D], zero where the row holds no latent.
    const int64_t dvp = dvp_;
    w_expand_ = rearranged(need(t, "v_up.weight"), (int64_t)H_ * dvp, D, [=](int64_t i, int64_t j) -> std::pair<int64_t, int64_t> {
                  const int64_t h = i / dvp, n = i % dvp;
                  if (n >= dv || j >= r) return {-1, 0};
                  return {h * dv + n, j};
                }).view({(int64_t)H_, dvp, D});
    w_o_ = pad_column_blocks(need(t, "o_proj.weight"), H_, dv_, dvp_);
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::Pages;
    n.num_kv_heads = 1;
    n.head_dim = D_;
    return n;
  }
  const char* step_inputs_key() const override { return "attention.items"; }
  void step_inputs(HostStep& step, std::vector<std::pair<std::string, HostArray>>& out) override {
    AttentionItems& m = attention_items(kernels, step);
    out.emplace_back("attention.prefill_items", m.prefill);
    out.emplace_back("attention.decode_items", m.decode);
  }
  int64_t workspace_floats(HostStep& step) override {
    AttentionItems& m = attention_items(kernels, step);
    return m.decode.shape[0] ? kernels.attn_scratch_floats((int)m.decode.shape[0], H_, D_, m.nseg) : 0;
  }
  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::Pages) throw EngineError("latent attention was handed a cache entry without pages");
    if (cache.writable != own_kv_) throw EngineError("latent attention: a layer writes the cache if and only if it has a latent projection of its own");
    Kernels& k = kernels;
    const int64_t T = x.dim(0);
    GroupTables& tables = ctx.groups.at(cache.group);
    const Tensor proj = k.gemm(x, w_in_);
    const Tensor q = k.gemm(k.norm_columns(proj, 0, rq_, q_norm_, eps_, rqp_), w_uq_);
    Tensor q_abs = k.empty({T, (int64_t)H_, (int64_t)D_});
    Tensor q_abs_rows = q_abs.view({T, (int64_t)H_ * D_});
    k.gemm_heads(q_abs_rows, D_, q, 0, qs_, w_absorb_);
    k.latent_post(proj, kv_col_, q, qs_, dp_, q_abs, &cache.k, &cache.v, cache.page_size, own_kv_ ? &kv_norm_ : nullptr, eps_,
                  *position_->angle_frequencies(), position_->pairs_neighbours(), ctx.positions, &tables.slots, r_, dr_);
    Tensor out = k.empty(q_abs.shape);
    AttentionItems& m = attention_items(k, *ctx.host);
    const Tensor& prefill_items = ctx.inputs.at("attention.prefill_items");
    const Tensor& decode_items = ctx.inputs.at("attention.decode_items");
    if (prefill_items.dim(0))
      k.paged_attention_capped(out, q_abs, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, prefill_items, 0, scale_, 0, 0, 0.f, nullptr,
                               ctx.host->k_len_bound, 0, nullptr, 0);
    if (decode_items.dim(0)) {
      const Tensor scratch = ctx.workspace(k.attn_scratch_floats((int)decode_items.dim(0), H_, D_, m.nseg));
      k.paged_attention_capped(out, q_abs, cache.k, cache.v, tables.block_table, ctx.cu_q, ctx.k_len, decode_items, 1, scale_, 0, 0, 0.f, nullptr,
                               m.decode_bound, m.nseg, &scratch, 0);
    }
    Tensor heads = k.empty({T, (int64_t)H_ * dvp_});
    k.gemm_heads(heads, dvp_, out.view({T, (int64_t)H_ * D_}), 0, D_, w_expand_);
    if (gate_) k.gate_mul(heads, proj, gate_col_, 0);
    return k.gemm(heads, w_o_);
  }

 private:
  int64_t hidden_;
  int H_, d_, dr_, dv_, r_, rq_, D_ = 0;       // D_: the head size of the cache and the attention kernels
  float scale_, eps_;
  bool own_kv_, gate_;
  int64_t dp_ = 0, qs_ = 0, rqp_ = 0, kvp_ = 0, dvp_ = 0, kv_col_ = -1, gate_col_ = 0;
  std::unique_ptr<PositionEncoding> position_;
  Tensor w_in_, w_uq_, w_absorb_, w_expand_, w_o_, q_norm_, kv_norm_;
};

// Linear attention with one fixed decay a head.  For the mixer's input h:
//   q = silu(W_q h), k = silu(W_k h) (heads x key size), v = silu(W_v h) (heads x value size);
//   per head, token by token:  S <- decay[head] S + k v^T;  o = S^T q  (no other scale);
//   y = norm(the heads' o side by side) (one root mean square over all of them, a weight of that width) * sigmoid(W_g h);
//   out = W_o y.
// A request's state slot holds the heads' S in 32-bit, zero at the request's start.  The four input projections are one
// launch, silu on its q, k and v columns a second; the recurrence is the delta rule's walk without its correction term, with
// the decays of the heads (numbers decay.0, decay.1, ...) in place of decays per token and channel; the read-out's norm and
// gate are one launch, a workgroup a row.
class FixedDecayAttention : public Mixer {
 public:
  FixedDecayAttention(const PartSpec& s, Kernels& k)
      : Mixer(k), hidden_(s.integer("hidden_size")), H_((int)s.integer("num_heads")), d_((int)s.integer("key_dim")), dv_((int)s.integer("value_dim")),
        eps_((float)s.number("eps")) {
    if (H_ < 1 || d_ < 1 || dv_ < 1 || d_ > 1024) throw ConfigError("linear attention: heads of " + std::to_string(d_) + " x " + std::to_string(dv_));
    std::vector<float> decay((size_t)H_);
    for (int h = 0; h < H_; ++h) decay[h] = (float)s.number("decay." + std::to_string(h));
    decay_ = zero_weight({(int64_t)H_}, DType::F32);
    hip_check(hipMemcpy(decay_.data, decay.data(), decay.size() * sizeof(float), hipMemcpyHostToDevice), "the heads' decays");
    qk_ = round_up((int64_t)H_ * d_, 8);
    v_ = round_up((int64_t)H_ * dv_, 8);
  }
  std::vector<ParamDecl> params() const override {
    const int64_t hd = (int64_t)H_ * d_, hv = (int64_t)H_ * dv_;
    ParamDecl q{"q_proj.weight", {hd, hidden_}}, kk{"k_proj.weight", {hd, hidden_}}, vv{"v_proj.weight", {hv, hidden_}};
    q.p0 = kk.p0 = vv.p0 = 0.1;
    ParamDecl norm{"out_norm.weight", {hv}, true, true, 0.9, 1.1};
    return {q, kk, vv, {"gate_proj.weight", {hv, hidden_}}, norm, {"o_proj.weight", {hidden_, hv}}};
  }
  void load(std::map<std::string, Tensor>& t) override {
    w_in_ = stack_rows({pad_matrix(need(t, "q_proj.weight"), qk_, hidden_), pad_matrix(need(t, "k_proj.weight"), qk_, hidden_),
                        pad_matrix(need(t, "v_proj.weight"), v_, hidden_), pad_matrix(need(t, "gate_proj.weight"), v_, hidden_)});
    out_norm_ = need(t, "out_norm.weight");
    w_o_ = pad_matrix(need(t, "o_proj.weight"), hidden_, v_);      // the read-out's width as whole 16-byte vectors
  }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {(int64_t)H_ * d_ * dv_};
    n.state_dtype = DType::F32;
    return n;
  }
  Tensor forward(const Tensor& x, StepContext& ctx, CacheEntry& cache) override {
    if (cache.kind != CacheNeed::State) throw EngineError("linear attention was handed a cache entry without state");
    Kernels& k = kernels;
    Tensor proj = k.gemm(x, w_in_);
    // q, k and v pass silu once, in place (the recurrence's workgroups would each do it again for the columns they share).
    k.silu_columns(proj, 0, 2 * qk_ + v_);
    const Tensor o = k.linear_rule(proj, 0, qk_, 2 * qk_, decay_, cache.state, ctx.cu_q, ctx.positions, ctx.state_slots, H_, d_, dv_, 1.f);
    return k.gemm(k.gated_row_norm(o, proj, 2 * qk_ + v_, out_norm_, eps_, 0, v_), w_o_);
  }

 private:
  int64_t hidden_;
  int H_, d_, dv_;
  float eps_;
  int64_t qk_ = 0, v_ = 0;
  Tensor w_in_, w_o_, out_norm_, decay_;
};

// What a layer adds from the token's own second embedding: with e the columns [first, first + n) of table[token],
//   g = gelu(W_gate x) * e;  y = W_out g;  the layer's norm 'side_out' then adds norm(y) to the stream.
// The table is one tensor for all layers that use it; n that is no whole 16-byte vector is padded with zeros in the weights.
class TokenSide : public Part {
 public:
  TokenSide(Kernels& k, int64_t hidden, int64_t vocab, int64_t n, int64_t first, int64_t table_width)
      : Part(k), hidden_(hidden), vocab_(vocab), n_(n), first_(first), width_(table_width) {
    if (n_ < 1 || first_ < 0 || first_ + n_ > width_) throw ConfigError("a token side input of " + std::to_string(n_) + " columns from " + std::to_string(first_) + " of " + std::to_string(width_));
  }
  std::vector<ParamDecl> params() const override {
    ParamDecl table{"table", {vocab_, width_}}, gate{"gate_proj.weight", {n_, hidden_}}, out{"out_proj.weight", {hidden_, n_}};
    table.p0 = 1.0;
    gate.p0 = 0.05;
    out.p0 = 0.2;
    return {table, gate, out};
  }
  void load(std::map<std::string, Tensor>& t) override {
    table_ = need(t, "table");
    const int64_t np = round_up(n_, 8);
    w_gate_ = pad_matrix(need(t, "gate_proj.weight"), np, hidden_);
    w_out_ = pad_matrix(need(t, "out_proj.weight"), hidden_, np);
  }
  // x: the stream as elements.
  Tensor forward(const Tensor& x, StepContext& ctx) {
    return kernels.gemm(kernels.side_gate(kernels.gemm(x, w_gate_), table_, ctx.ids, first_, n_), w_out_);
  }

 private:
  int64_t hidden_, vocab_, n_, first_, width_;
  Tensor table_, w_gate_, w_out_;
};

// A residual stream x in 32-bit whose sublayers read it as it is (rounded to elements), with a norm on their outputs only:
//   x <- x + norm_mixer_out(mixer(x));  x <- x + norm_ffn_out(ffn(x)) (if the layer has a feed-forward);
//   x <- x + norm_side_out(side(x, token)) (if the numbers side_dim, side_first, side_width and vocab_size are given:
//   TokenSide above).
class PostNormBlock : public Block {
 public:
  PostNormBlock(Kernels& k, std::unique_ptr<Mixer> mixer, std::unique_ptr<FeedForward> ffn, std::map<std::string, std::unique_ptr<Norm>> norms,
                const std::map<std::string, double>& numbers)
      : Block(k), mixer_(std::move(mixer)), ffn_(std::move(ffn)), norms_(std::move(norms)) {
    auto number = [&](const char* name) {
      auto it = numbers.find(name);
      if (it == numbers.end()) throw ConfigError(std::string("a post_norm block needs the number '") + name + "'");
      return (int64_t)it->second;
    };
    hidden_ = number("hidden_size");
    has_ffn_ = dynamic_cast<NoFeedForward*>(ffn_.get()) == nullptr;
    if (!norms_.count("mixer_out")) throw ConfigError("a post_norm block needs the norm 'mixer_out'");
    if (has_ffn_ && !norms_.count("ffn_out")) throw ConfigError("a post_norm block with a feed-forward needs the norm 'ffn_out'");
    if (numbers.count("side_dim")) {
      if (!norms_.count("side_out")) throw ConfigError("a post_norm block with a token side input needs the norm 'side_out'");
      side_.reset(new TokenSide(k, hidden_, number("vocab_size"), number("side_dim"), number("side_first"), number("side_width")));
    }
  }
  std::vector<std::pair<std::string, Part*>> children() override {
    std::vector<std::pair<std::string, Part*>> c = {{"mixer", mixer_.get()}, {"feed_forward", ffn_.get()}};
    for (auto& n : norms_) c.emplace_back("norms." + n.first, n.second.get());
    if (side_) c.emplace_back("side", side_.get());
    return c;
  }
  Mixer& mixer() override { return *mixer_; }
  std::pair<Tensor, Tensor> forward(const Tensor& hidden, Tensor residual, StepContext& ctx, CacheEntry& cache) override {
    Kernels& k = kernels;
    if (hidden.dtype != DType::F32 || hidden.shape.size() != 2 || hidden.dim(1) != hidden_)
      throw EngineError("a post_norm block takes the 32-bit residual stream, not " + hidden.describe());
    Tensor stream = hidden;
    // What the next sublayer reads, the stream rounded to elements, is written by the launch that adds to the stream; the
    // layer's first sublayer finds what the layer before left (ctx.carry), or rounds the stream itself.  Where the elements
    // are 32-bit the stream is read as it is.
    const bool narrow = k.dtype() != DType::F32;
    Tensor read;
    auto left = ctx.carry.find("stream.rounded");
    if (!narrow) read = stream;
    else if (left != ctx.carry.end() && ctx.carry["stream.rounded_of"].data == stream.data && left->second.shape == stream.shape) read = left->second;
    else read = k.to_elements(stream);
    auto add = [&](const char* norm, const Tensor& y) {
      if (!narrow) {
        norms_[norm]->forward_scaled_add(y, stream, stream, 1.f);
        return;
      }
      read = k.empty(stream.shape);
      norms_[norm]->forward_scaled_add(y, stream, stream, 1.f, &read);
    };
    add("mixer_out", mixer_->forward(read, ctx, cache));
    if (has_ffn_) add("ffn_out", ffn_->forward(read, ctx));
    if (side_) add("side_out", side_->forward(read, ctx));
    if (narrow) {
      ctx.carry["stream.rounded"] = read;
      ctx.carry["stream.rounded_of"] = stream;
    }
    return {stream, residual};
  }

 private:
  std::unique_ptr<Mixer> mixer_;
  std::unique_ptr<FeedForward> ffn_;
  std::map<std::string, std::unique_ptr<Norm>> norms_;
  std::unique_ptr<TokenSide> side_;
  int64_t hidden_ = 0;
  bool has_ffn_ = true;
};

template <class T>
PartFactory factory() {
  return [](const PartSpec& s, Kernels& k) { return std::unique_ptr<Part>(new T(s, k)); };
}

}  // namespace

void register_standard_parts() {
  static std::once_flag once;
  std::call_once(once, [] {
    register_part("embedding", "token_embedding", factory<TokenEmbedding>());
    register_part("embedding", "token_embedding_sinusoid", factory<SinusoidEmbedding>());
    register_part("mixer", "channel_delta", factory<ChannelDelta>());
    register_part("feed_forward", "none", factory<NoFeedForward>());
    register_block("sandwich_depth", [](Kernels& k, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                        std::map<std::string, std::unique_ptr<Norm>> n, const std::map<std::string, double>& numbers) {
      return std::unique_ptr<Block>(new SandwichDepthBlock(k, std::move(m), std::move(f), std::move(n), numbers));
    });
    register_block("sandwich", [](Kernels& k, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                  std::map<std::string, std::unique_ptr<Norm>> n, const std::map<std::string, double>& numbers) {
      std::map<std::string, double> plain = numbers;
      plain.erase("states");
      plain.erase("depth");
      return std::unique_ptr<Block>(new SandwichDepthBlock(k, std::move(m), std::move(f), std::move(n), plain));
    });
    register_part("mixer", "gated_linear_attention", factory<GatedLinearAttention>());
    register_part("embedding", "token_embedding_scaled", factory<ScaledEmbedding>());
    register_part("position", "rotary_stretched", factory<RotaryStretched>());
    register_part("mixer", "state_space", factory<StateSpace>());
    register_part("mixer", "pair_mean", factory<PairMean>());
    register_part("feed_forward", "routed_experts", factory<RoutedExperts>());
    register_block("parallel_sum", [](Kernels& k, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                      std::map<std::string, std::unique_ptr<Norm>> n, const std::map<std::string, double>& numbers) {
      return std::unique_ptr<Block>(new ParallelSumBlock(k, std::move(m), std::move(f), std::move(n), numbers));
    });
    register_part("mixer", "latent_attention", factory<LatentAttention>());
    register_part("mixer", "fixed_decay_attention", factory<FixedDecayAttention>());
    register_block("post_norm", [](Kernels& k, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                   std::map<std::string, std::unique_ptr<Norm>> n, const std::map<std::string, double>& numbers) {
      return std::unique_ptr<Block>(new PostNormBlock(k, std::move(m), std::move(f), std::move(n), numbers));
    });
    register_part("norm", "rmsnorm", factory<RMSNorm>());
    register_part("position", "rotary", factory<Rotary>());
    register_part("mixer", "attention", factory<Attention>());
    register_part("feed_forward", "swiglu", factory<SwiGLU>());
    register_part("head", "linear_head", factory<LinearHead>());
    register_block("prenorm", [](Kernels& k, std::unique_ptr<Mixer> m, std::unique_ptr<FeedForward> f,
                                 std::map<std::string, std::unique_ptr<Norm>> n, const std::map<std::string, double>&) {
      return std::unique_ptr<Block>(new PreNormBlock(k, std::move(m), std::move(f), std::move(n)));
    });
  });
}

}  // namespace vosti
