#include "pabavik.h"

#include <cmath>

namespace vosti {
namespace {

PartSpecPtr make(std::string kind, std::map<std::string, double> numbers, std::map<std::string, PartSpecPtr> parts = {}) {
  auto p = std::make_shared<PartSpec>();
  p->kind = std::move(kind);
  p->numbers = std::move(numbers);
  for (auto& c : parts) p->parts[c.first] = c.second;
  return p;
}

const Json* present(const Json& j, const std::string& key) {
  const Json* v = j.get(key);
  return v && v->kind != Json::Null ? v : nullptr;
}

const Json& member(const Json& j, const std::string& key, const std::string& where) {
  const Json* v = present(j, key);
  if (!v) throw ConfigError("config.json: " + where + " lacks '" + key + "'");
  return *v;
}

int64_t positive(const Json& j, const std::string& key, const std::string& where) {
  const Json& v = member(j, key, where);
  if (!v.is_int() || v.as_int() <= 0) throw ConfigError("config.json: " + where + " '" + key + "' must be a positive integer");
  return v.as_int();
}

double finite(const Json& j, const std::string& key, const std::string& where) {
  const Json& v = member(j, key, where);
  if (v.kind != Json::Number || !std::isfinite(v.number)) throw ConfigError("config.json: " + where + " '" + key + "' must be a finite number");
  return v.number;
}

}  // namespace

// The constants that the design fixes stand here; everything else is read from the configuration.
constexpr double kGluSlope = 1.702;         // an expert's gate is g * sigmoid(this * g)
constexpr double kGluUpShift = 1.0;         // and multiplies (u + this)
constexpr int64_t kMaxPositions = 1 << 22;  // the angles are computed, not tabulated; this bounds a request's length

// Softmax attention over a window, on keys of its own or of the layer `kv_from` names.
static PartSpecPtr attention_mixer(const Json& m, int64_t width, double eps, int64_t layer, const std::string& where, const std::string& p, LayerSpec& ls,
                                   int& cache_from) {
  const int64_t heads = positive(m, "heads", where), kv_heads = positive(m, "kv_heads", where);
  const int64_t dim = positive(m, "dim", where), vdim = positive(m, "vdim", where);
  if (heads % kv_heads) throw ConfigError("config.json: " + where + ": 'heads' must be a multiple of 'kv_heads'");
  const double scale = finite(m, "scale", where);
  if (scale <= 0) throw ConfigError("config.json: " + where + ": 'scale' must be positive");
  const int64_t window = positive(member(m, "mask", where), "size", where + " mask");
  const Json& rot = member(m, "rot", where);
  const int64_t dims = positive(rot, "dims", where + " rot");
  const double base = finite(rot, "base", where + " rot");
  if (dims % 2 || dims > dim) throw ConfigError("config.json: " + where + ": 'rot.dims' must be even and at most 'dim'");
  if (base <= 1.0) throw ConfigError("config.json: " + where + ": 'rot.base' must be larger than 1");
  cache_from = -1;
  if (const Json* from = present(m, "kv_from")) {
    if (!from->is_int() || from->as_int() < 0 || from->as_int() >= layer)
      throw ConfigError("config.json: " + where + ": 'kv_from' must name an earlier layer");
    cache_from = (int)from->as_int();
  }
  const PartSpecPtr head_norm = make("rmsnorm", {{"size", (double)dim}, {"eps", eps}});
  std::map<std::string, PartSpecPtr> below = {
      {"q_norm", head_norm},
      {"position", make("rotary_stretched", {{"head_dim", (double)dim}, {"rotary_dim", (double)dims}, {"theta", base}, {"max_positions", (double)kMaxPositions}})}};
  ls.names["mixer.q_proj.weight"] = p + "mix.q";
  ls.names["mixer.q_norm.weight"] = p + "mix.q.norm";
  ls.names["mixer.gate_proj.weight"] = p + "mix.g";
  ls.names["mixer.o_proj.weight"] = p + "mix.o";
  if (cache_from < 0) {
    below["k_norm"] = head_norm;
    ls.names["mixer.k_proj.weight"] = p + "mix.k";
    ls.names["mixer.k_norm.weight"] = p + "mix.k.norm";
    ls.names["mixer.v_proj.weight"] = p + "mix.v";
  }
  // sink 2: the softmax's denominator holds one more term, exp(0), that has no key and no value.
  return make("attention", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"num_kv_heads", (double)kv_heads},
                            {"head_dim", (double)dim}, {"value_dim", (double)vdim}, {"scale", scale}, {"window", (double)window},
                            {"sink", 2.0}, {"exact_weights", 1.0}, {"own_kv", cache_from < 0 ? 1.0 : 0.0}, {"output_gate", 1.0}},
              below);
}

// Gated linear attention with a decay per key channel.
static PartSpecPtr linear_mixer(const Json& m, int64_t width, double eps, const std::string& where, const std::string& p, LayerSpec& ls) {
  const int64_t heads = positive(m, "heads", where), dim = positive(m, "dim", where), vdim = positive(m, "vdim", where);
  const double tau = finite(m, "tau", where);
  if (tau <= 0) throw ConfigError("config.json: " + where + ": 'tau' must be positive");
  const std::pair<const char*, const char*> names[] = {{"q_proj.weight", "q"},       {"k_proj.weight", "k"},      {"v_proj.weight", "v"},
                                                       {"gate_proj.weight", "g"},    {"o_proj.weight", "o"},      {"out_norm.weight", "norm"},
                                                       {"decay_down.weight", "a1"},  {"decay_up.weight", "a2"},   {"decay_up.bias", "a2.b"}};
  for (const auto& n : names) ls.names[std::string("mixer.") + n.first] = p + "mix." + n.second;
  // The rank of the decay's two projections is in no key: the stored tensors give it.
  return make("gated_linear_attention", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"key_dim", (double)dim},
                                         {"value_dim", (double)vdim}, {"decay_root", tau}, {"eps", eps}});
}

// One expert's sizes and limit from its entry.
static void expert_numbers(const Json& e, const std::string& where, int64_t& ff, double& limit) {
  ff = positive(e, "ff", where);
  limit = finite(e, "limit", where);
  if (limit <= 0) throw ConfigError("config.json: " + where + ": 'limit' must be positive");
}

ModelSpec pabavik_model_spec(const Json& raw) {
  const int64_t width = positive(raw, "width", "the model's"), vocab = positive(raw, "vocab", "the model's");
  const double eps = finite(member(raw, "norm", "the model"), "eps", "norm");
  if (eps < 0) throw ConfigError("config.json: 'norm.eps' must not be negative");
  const double embed_scale = finite(member(raw, "embedding", "the model"), "scale", "embedding");
  const double logit_cap = present(raw, "logit_softcap") ? finite(raw, "logit_softcap", "the model's") : 0.0;
  if (logit_cap < 0) throw ConfigError("config.json: 'logit_softcap' must not be negative");
  const Json& layers = member(raw, "layers", "the model");
  if (layers.kind != Json::Array) throw ConfigError("config.json: 'layers' must be a list");
  const int64_t L = (int64_t)layers.items.size();
  const PartSpecPtr norm = make("rmsnorm", {{"size", (double)width}, {"eps", eps}, {"offset", 1.0}});

  ModelSpec spec;
  spec.architecture = "Pabavik";
  spec.vocab_size = vocab;
  spec.hidden_size = width;
  spec.max_positions = kMaxPositions;
  spec.embedding = make("token_embedding_scaled", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}, {"scale", embed_scale}});
  spec.final_norm = norm;
  spec.head = make("linear_head", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}, {"softcap", logit_cap}});
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers.items[i];
    const std::string where = "layer " + std::to_string(i);
    const std::string p = "l" + std::to_string(i) + ".";
    const Json* type = l.get("type");
    if (!type || type->kind != Json::String) throw ConfigError("config.json: " + where + " lacks 'type'");
    const Json& m = member(l, "mixer", where);
    LayerSpec ls;
    ls.block = "sandwich";
    ls.block_numbers = {{"residual_mult", 1.0}, {"hidden_size", (double)width}};
    ls.norms = {{"mixer_in", norm}, {"mixer_out", norm}};
    ls.names = {{"norms.mixer_in.weight", p + "norm1"}, {"norms.mixer_out.weight", p + "norm1b"}};
    int cache_from = -1;
    if (type->text == "attention") ls.mixer = attention_mixer(m, width, eps, i, where, p, ls, cache_from);
    else if (type->text == "gla") ls.mixer = linear_mixer(m, width, eps, where, p, ls);
    else throw ConfigError("config.json: " + where + ": unknown mixer type '" + type->text + "'");
    if (cache_from >= 0) {
      // The layer that lends its keys has projections of its own, and the same heads and rotation.
      const Json* src_type = layers.items[cache_from].get("type");
      const Json* src = present(layers.items[cache_from], "mixer");
      if (!src_type || src_type->kind != Json::String || src_type->text != "attention" || !src || present(*src, "kv_from"))
        throw ConfigError("config.json: " + where + ": 'kv_from' must name an attention layer with keys of its own");
      for (const char* key : {"kv_heads", "dim", "vdim"})
        if (positive(*src, key, "layer " + std::to_string(cache_from)) != positive(m, key, where))
          throw ConfigError("config.json: " + where + ": '" + key + "' differs from the layer whose keys it reads");
    }
    if (const Json* mlp = present(l, "mlp")) {
      const std::string mw = where + " mlp";
      const Json* kind = mlp->get("kind");
      // The design has one kind of feed-forward; a configuration that names none means that one.
      if (kind && kind->kind != Json::Null && (kind->kind != Json::String || kind->text != "moe"))
        throw ConfigError("config.json: " + where + ": the feed-forward's 'kind' must be 'moe'");
      const Json& router = member(*mlp, "router", mw);
      const int64_t experts = positive(router, "experts", mw + ".router"), top = positive(router, "top", mw + ".router");
      if (top > experts) throw ConfigError("config.json: " + where + ": 'top' must not exceed 'experts'");
      int64_t ff = 0, shared_ff = 0;
      double limit = 0, shared_limit = 0;
      expert_numbers(member(*mlp, "expert", mw), mw + ".expert", ff, limit);
      std::map<std::string, double> n = {{"hidden_size", (double)width}, {"intermediate_size", (double)ff}, {"experts", (double)experts},
                                         {"top", (double)top}, {"router_bias", 1.0}, {"gated", 1.0}, {"limit", limit},
                                         {"glu_slope", kGluSlope}, {"up_shift", kGluUpShift}};
      ls.names["feed_forward.router.weight"] = p + "mlp.router";
      ls.names["feed_forward.router.bias"] = p + "mlp.router.b";
      for (int64_t e = 0; e < experts; ++e) {
        const std::string en = std::to_string(e);
        for (const char* w : {"gate", "up", "down"}) ls.names["feed_forward.experts." + en + "." + w + "_proj.weight"] = p + "mlp.e" + en + "." + w;
      }
      if (const Json* shared = present(*mlp, "shared")) {
        expert_numbers(*shared, mw + ".shared", shared_ff, shared_limit);
        n["shared_size"] = (double)shared_ff;
        n["shared_limit"] = shared_limit;
        for (const char* w : {"gate", "up", "down"}) ls.names[std::string("feed_forward.shared.") + w + "_proj.weight"] = p + "mlp.shared." + w;
      }
      ls.feed_forward = make("routed_experts", n);
      ls.norms["ffn_in"] = norm;
      ls.norms["ffn_out"] = norm;
      ls.names["norms.ffn_in.weight"] = p + "norm2";
      ls.names["norms.ffn_out.weight"] = p + "norm2b";
    } else {
      ls.feed_forward = make("none", {});
      // The layer's second pair of norms has nothing to stand around; a checkpoint may still hold their weights.
      spec.ignored_names.push_back(p + "norm2");
      spec.ignored_names.push_back(p + "norm2b");
    }
    spec.layers.push_back(std::move(ls));
    spec.schedule.push_back({(int)i, cache_from});
  }
  spec.names = {{"embedding.weight", "embed"}, {"final_norm.weight", "final.norm"}, {"head.weight", "head"}};
  spec.config_json = "{\"vocab\": " + std::to_string(vocab) + ", \"width\": " + std::to_string(width) + ", \"layers\": " + std::to_string(L) +
                     ", \"embedding_scale\": " + json_number(embed_scale) + ", \"norm_eps\": " + json_number(eps) + ", \"logit_softcap\": " +
                     json_number(logit_cap) + "}";
  return spec;
}

}  // namespace vosti
