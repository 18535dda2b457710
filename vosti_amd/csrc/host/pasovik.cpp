#include "pasovik.h"

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

// The constants that the design fixes stand here; everything else is read from the configuration.
constexpr double kGluSlope = 1.702;         // an expert's gate is g * sigmoid(this * g)
constexpr double kGluUpShift = 1.0;         // and multiplies (u + this)
constexpr int64_t kMaxPositions = 1 << 22;  // the angles are computed, not tabulated; this bounds a request's length

// A rotation of neighbouring pairs by computed angles: entries 2i and 2i + 1 of the first `dims` of a head turn by
// position * base^(-2i/dims) / factor (no 'scaling': factor 1).
PartSpecPtr rotation(const Json& rot, int64_t head_dim, const std::string& where) {
  const int64_t dims = positive(rot, "dims", where + " rot");
  const double base = finite(rot, "base", where + " rot");
  if (dims % 2 || dims > head_dim) throw ConfigError("config.json: " + where + ": 'rot.dims' must be even and at most the size it rotates");
  if (base <= 1.0) throw ConfigError("config.json: " + where + ": 'rot.base' must be larger than 1");
  double factor = 1.0;
  if (const Json* scaling = present(rot, "scaling")) {
    factor = finite(*scaling, "factor", where + " rot.scaling");
    if (factor <= 0) throw ConfigError("config.json: " + where + ": 'rot.scaling.factor' must be positive");
  }
  return make("rotary_stretched", {{"head_dim", (double)head_dim}, {"rotary_dim", (double)dims}, {"theta", base}, {"linear_factor", factor},
                                   {"neighbours", 1.0}, {"max_positions", (double)kMaxPositions}});
}

// Softmax attention over all earlier keys.
PartSpecPtr attention_mixer(const Json& m, int64_t width, double eps, const std::string& where, const std::string& p, LayerSpec& ls) {
  const int64_t heads = positive(m, "heads", where), kv_heads = positive(m, "kv_heads", where);
  const int64_t dim = positive(m, "dim", where), vdim = positive(m, "vdim", where);
  if (heads % kv_heads) throw ConfigError("config.json: " + where + ": 'heads' must be a multiple of 'kv_heads'");
  const double scale = finite(m, "scale", where);
  if (scale <= 0) throw ConfigError("config.json: " + where + ": 'scale' must be positive");
  const double softcap = present(m, "softcap") ? finite(m, "softcap", where) : 0.0;
  if (softcap < 0) throw ConfigError("config.json: " + where + ": 'softcap' must not be negative");
  const PartSpecPtr head_norm = make("rmsnorm", {{"size", (double)dim}, {"eps", eps}});
  std::map<std::string, PartSpecPtr> below = {{"q_norm", head_norm}, {"k_norm", head_norm}, {"position", rotation(member(m, "rot", where), dim, where)}};
  const std::pair<const char*, const char*> names[] = {{"q_proj.weight", "q"}, {"k_proj.weight", "k"},      {"v_proj.weight", "v"},
                                                       {"o_proj.weight", "o"}, {"q_norm.weight", "q.norm"}, {"k_norm.weight", "k.norm"}};
  for (const auto& n : names) ls.names[std::string("mixer.") + n.first] = p + "mix." + n.second;
  return make("attention", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"num_kv_heads", (double)kv_heads}, {"head_dim", (double)dim},
                            {"value_dim", (double)vdim}, {"scale", scale}, {"softcap", softcap}, {"exact_weights", 1.0}},
              below);
}

// Attention through a latent, on a latent of its own or on that of the layer `kv_from` names.
PartSpecPtr latent_mixer(const Json& m, int64_t width, double eps, int64_t layer, const std::string& where, const std::string& p, LayerSpec& ls,
                         int& cache_from) {
  const int64_t heads = positive(m, "heads", where), dim = positive(m, "dim", where), rot_dim = positive(m, "rot_dim", where);
  const int64_t vdim = positive(m, "vdim", where), kv_rank = positive(m, "kv_rank", where), q_rank = positive(m, "q_rank", where);
  const double scale = finite(m, "scale", where);
  if (scale <= 0) throw ConfigError("config.json: " + where + ": 'scale' must be positive");
  const PartSpecPtr position = rotation(member(m, "rot", where), rot_dim, where);
  if (position->integer("rotary_dim") != rot_dim) throw ConfigError("config.json: " + where + ": 'rot.dims' must equal 'rot_dim'");
  cache_from = -1;
  if (const Json* from = present(m, "kv_from")) {
    if (!from->is_int() || from->as_int() < 0 || from->as_int() >= layer)
      throw ConfigError("config.json: " + where + ": 'kv_from' must name an earlier layer");
    cache_from = (int)from->as_int();
  }
  std::vector<std::pair<const char*, const char*>> names = {{"q_down.weight", "dq"},   {"q_down_norm.weight", "dq.norm"}, {"q_up.weight", "uq"},
                                                            {"k_up.weight", "uk"},     {"v_up.weight", "uv"},             {"gate_proj.weight", "g"},
                                                            {"o_proj.weight", "o"}};
  if (cache_from < 0) {
    names.push_back({"kv_down.weight", "dkv"});
    names.push_back({"kv_down_norm.weight", "dkv.norm"});
  }
  for (const auto& n : names) ls.names[std::string("mixer.") + n.first] = p + "mix." + n.second;
  return make("latent_attention", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"head_dim", (double)dim}, {"rotary_dim", (double)rot_dim},
                                   {"value_dim", (double)vdim}, {"kv_rank", (double)kv_rank}, {"q_rank", (double)q_rank}, {"scale", scale},
                                   {"eps", eps}, {"own_kv", cache_from < 0 ? 1.0 : 0.0}, {"output_gate", 1.0}},
              {{"position", position}});
}

// Linear attention with a fixed decay per head.
PartSpecPtr linear_mixer(const Json& m, int64_t width, double eps, const std::string& where, const std::string& p, LayerSpec& ls) {
  const int64_t heads = positive(m, "heads", where), dim = positive(m, "dim", where), vdim = positive(m, "vdim", where);
  const Json& decay = member(m, "decay", where);
  if (decay.kind != Json::Array || (int64_t)decay.items.size() != heads) throw ConfigError("config.json: " + where + ": 'decay' must list one number a head");
  std::map<std::string, double> n = {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"key_dim", (double)dim}, {"value_dim", (double)vdim},
                                     {"eps", eps}};
  for (int64_t h = 0; h < heads; ++h) {
    const Json& d = decay.items[h];
    if (d.kind != Json::Number || !std::isfinite(d.number) || d.number < 0 || d.number > 1)
      throw ConfigError("config.json: " + where + ": a decay must lie between 0 and 1");
    n["decay." + std::to_string(h)] = d.number;
  }
  for (const char* t : {"q", "k", "v"}) ls.names[std::string("mixer.") + t + "_proj.weight"] = p + "mix." + t;
  ls.names["mixer.gate_proj.weight"] = p + "mix.g";
  ls.names["mixer.o_proj.weight"] = p + "mix.o";
  ls.names["mixer.out_norm.weight"] = p + "mix.norm";
  return make("fixed_decay_attention", n);
}

}  // namespace

ModelSpec pasovik_model_spec(const Json& raw) {
  const int64_t width = positive(raw, "width", "the model's"), vocab = positive(raw, "vocab", "the model's");
  const double eps = finite(member(raw, "norm", "the model"), "eps", "norm");
  if (eps < 0) throw ConfigError("config.json: 'norm.eps' must not be negative");
  const Json& layers = member(raw, "layers", "the model");
  if (layers.kind != Json::Array) throw ConfigError("config.json: 'layers' must be a list");
  const int64_t L = (int64_t)layers.items.size();
  const int64_t side = present(raw, "token_side") ? positive(*present(raw, "token_side"), "dim", "token_side") : 0;
  const PartSpecPtr norm = make("rmsnorm", {{"size", (double)width}, {"eps", eps}});

  ModelSpec spec;
  spec.architecture = "Pasovik";
  spec.vocab_size = vocab;
  spec.hidden_size = width;
  spec.max_positions = kMaxPositions;
  spec.embedding = make("token_embedding_scaled", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}, {"scale", 1.0}});
  spec.final_norm = norm;
  spec.head = make("linear_head", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}});
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers.items[i];
    const std::string where = "layer " + std::to_string(i);
    const std::string p = "l" + std::to_string(i) + ".";
    const Json* type = l.get("type");
    if (!type || type->kind != Json::String) throw ConfigError("config.json: " + where + " lacks 'type'");
    const Json& m = member(l, "mixer", where);
    LayerSpec ls;
    ls.block = "post_norm";
    ls.block_numbers = {{"hidden_size", (double)width}};
    ls.norms = {{"mixer_out", norm}};
    ls.names = {{"norms.mixer_out.weight", p + "norm1"}};
    int cache_from = -1;
    if (type->text == "attention") ls.mixer = attention_mixer(m, width, eps, where, p, ls);
    else if (type->text == "latent_attention") ls.mixer = latent_mixer(m, width, eps, i, where, p, ls, cache_from);
    else if (type->text == "lightning") ls.mixer = linear_mixer(m, width, eps, where, p, ls);
    else throw ConfigError("config.json: " + where + ": unknown mixer type '" + type->text + "'");
    if (cache_from >= 0) {
      // The layer that lends its latent has a projection of its own, and the same latent, rotated part and rotation.
      const Json* src_type = layers.items[cache_from].get("type");
      const Json* src = present(layers.items[cache_from], "mixer");
      if (!src_type || src_type->kind != Json::String || src_type->text != "latent_attention" || !src || present(*src, "kv_from"))
        throw ConfigError("config.json: " + where + ": 'kv_from' must name a latent attention layer with a latent of its own");
      for (const char* key : {"kv_rank", "rot_dim"})
        if (positive(*src, key, "layer " + std::to_string(cache_from)) != positive(m, key, where))
          throw ConfigError("config.json: " + where + ": '" + key + "' differs from the layer whose latent it reads");
      const PartSpecPtr theirs = rotation(member(*src, "rot", where), positive(*src, "rot_dim", where), where);
      if (theirs->numbers != ls.mixer->part("position")->numbers)
        throw ConfigError("config.json: " + where + ": the rotation differs from the layer whose latent it reads");
    }
    if (const Json* mlp = present(l, "mlp")) {
      const std::string mw = where + " mlp";
      const Json* kind = mlp->get("kind");
      if (!kind || kind->kind != Json::String || (kind->text != "dense" && kind->text != "moe"))
        throw ConfigError("config.json: " + where + ": the feed-forward's 'kind' must be 'dense' or 'moe'");
      if (kind->text == "dense") {
        ls.feed_forward = make("swiglu", {{"hidden_size", (double)width}, {"intermediate_size", (double)positive(*mlp, "ff", mw)}});
        for (const char* w : {"gate", "up", "down"}) ls.names[std::string("feed_forward.") + w + "_proj.weight"] = p + "mlp." + w;
      } else {
        const Json& router = member(*mlp, "router", mw);
        const int64_t experts = positive(router, "experts", mw + ".router"), top = positive(router, "top", mw + ".router");
        if (top > experts) throw ConfigError("config.json: " + where + ": 'top' must not exceed 'experts'");
        const Json& expert = member(*mlp, "expert", mw);
        const int64_t ff = positive(expert, "ff", mw + ".expert");
        const double limit = finite(expert, "limit", mw + ".expert");
        if (limit <= 0) throw ConfigError("config.json: " + where + ": 'limit' must be positive");
        // score 1: the weights are the logistic function of the chosen logits, as they are; weigh_input: a weight scales
        // what its expert reads, not what it gives.
        ls.feed_forward = make("routed_experts", {{"hidden_size", (double)width}, {"intermediate_size", (double)ff}, {"experts", (double)experts},
                                                  {"top", (double)top}, {"gated", 1.0}, {"limit", limit}, {"glu_slope", kGluSlope},
                                                  {"up_shift", kGluUpShift}, {"score", 1.0}, {"weigh_input", 1.0}});
        ls.names["feed_forward.router.weight"] = p + "mlp.router";
        for (int64_t e = 0; e < experts; ++e) {
          const std::string en = std::to_string(e);
          for (const char* w : {"gate", "up", "down"}) ls.names["feed_forward.experts." + en + "." + w + "_proj.weight"] = p + "mlp.e" + en + "." + w;
        }
      }
      ls.norms["ffn_out"] = norm;
      ls.names["norms.ffn_out.weight"] = p + "norm2";
    } else {
      ls.feed_forward = make("none", {});
      spec.ignored_names.push_back(p + "norm2");      // nothing to stand behind; a checkpoint may still hold the weight
    }
    if (side > 0) {
      // The layer's slice of the token's second embedding: columns [i * side, (i + 1) * side) of a table all layers share.
      ls.block_numbers["side_dim"] = (double)side;
      ls.block_numbers["side_first"] = (double)(i * side);
      ls.block_numbers["side_width"] = (double)(L * side);
      ls.block_numbers["vocab_size"] = (double)vocab;
      ls.norms["side_out"] = norm;
      ls.names["norms.side_out.weight"] = p + "side.norm";
      ls.names["side.table"] = "side.embed";
      ls.names["side.gate_proj.weight"] = p + "side.gate";
      ls.names["side.out_proj.weight"] = p + "side.proj";
    }
    spec.layers.push_back(std::move(ls));
    spec.schedule.push_back({(int)i, cache_from});
  }
  spec.names = {{"embedding.weight", "embed"}, {"final_norm.weight", "final.norm"}, {"head.weight", "head"}};
  spec.config_json = "{\"vocab\": " + std::to_string(vocab) + ", \"width\": " + std::to_string(width) + ", \"layers\": " + std::to_string(L) +
                     ", \"norm_eps\": " + json_number(eps) + ", \"token_side\": " + std::to_string(side) + "}";
  return spec;
}

}  // namespace vosti
