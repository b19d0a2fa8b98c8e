#include "povatar.h"

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

const Json& member(const Json& j, const std::string& key, const std::string& where) {
  const Json* v = j.get(key);
  if (!v || v->kind == Json::Null) throw ConfigError("config.json: " + where + " lacks '" + key + "'");
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

const Json* present(const Json& j, const std::string& key) {
  const Json* v = j.get(key);
  return v && v->kind != Json::Null ? v : nullptr;
}

}  // namespace

// The constants that the design fixes stand here; everything else is read from the configuration.
constexpr double kRouterWeightEps = 1e-20;   // the chosen experts' scores are divided by their sum plus this
constexpr int64_t kMaxPositions = 1 << 22;   // the angles are computed, not tabulated; this bounds a request's length

// The softmax attention of a layer's left half.
static PartSpecPtr left_mixer(const Json& m, int64_t width, const std::string& where, const std::string& p, LayerSpec& ls) {
  const int64_t heads = positive(m, "heads", where), kv_heads = positive(m, "kv_heads", where);
  const int64_t dim = positive(m, "dim", where), vdim = positive(m, "vdim", where);
  if (heads % kv_heads) throw ConfigError("config.json: " + where + ": 'heads' must be a multiple of 'kv_heads'");
  const double scale = finite(m, "scale", where);
  if (scale <= 0) throw ConfigError("config.json: " + where + ": 'scale' must be positive");
  int64_t block = 0;
  if (const Json* mask = present(m, "mask")) block = positive(*mask, "size", where + " mask");
  std::map<std::string, PartSpecPtr> below;
  if (const Json* rot = present(m, "rot")) {
    const int64_t dims = positive(*rot, "dims", where + " rot");
    if (dims % 2 || dims > dim) throw ConfigError("config.json: " + where + ": 'rot.dims' must be even and at most 'dim'");
    std::map<std::string, double> n = {{"head_dim", (double)dim}, {"rotary_dim", (double)dims}, {"theta", finite(*rot, "base", where + " rot")},
                                       {"max_positions", (double)kMaxPositions}};
    if (n["theta"] <= 1.0) throw ConfigError("config.json: " + where + ": 'rot.base' must be larger than 1");
    if (const Json* s = present(*rot, "scaling")) {
      const std::string w = where + " rot.scaling";
      n["factor"] = finite(*s, "factor", w);
      n["original"] = finite(*s, "original", w);
      n["fast"] = finite(*s, "fast", w);
      n["slow"] = finite(*s, "slow", w);
      if (n["factor"] <= 0 || n["original"] <= 0 || n["fast"] <= 0 || n["slow"] <= 0)
        throw ConfigError("config.json: " + w + ": 'factor', 'original', 'fast' and 'slow' must be positive");
    }
    below["position"] = make("rotary_stretched", n);
  }
  for (const char* n : {"q", "k", "v", "o"}) ls.names[std::string("mixer.left.") + n + "_proj.weight"] = p + "mix.left." + n;
  // sink 2: the softmax's denominator holds one more term, exp(0), that has no key and no value.
  return make("attention", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"num_kv_heads", (double)kv_heads},
                            {"head_dim", (double)dim}, {"value_dim", (double)vdim}, {"scale", scale}, {"block", (double)block},
                            {"sink", 2.0}, {"exact_weights", 1.0}},
              below);
}

// The state-space recurrence of a layer's right half.
static PartSpecPtr right_mixer(const Json& m, int64_t width, double eps, const std::string& where, const std::string& p, LayerSpec& ls) {
  const int64_t heads = positive(m, "heads", where), vdim = positive(m, "vdim", where), state = positive(m, "state", where);
  const int64_t groups = positive(m, "groups", where), parts = positive(m, "norm_groups", where), taps = positive(m, "conv", where);
  if (heads % groups) throw ConfigError("config.json: " + where + ": 'heads' must be a multiple of 'groups'");
  if ((heads * vdim) % parts) throw ConfigError("config.json: " + where + ": 'norm_groups' must divide heads * vdim");
  const std::pair<const char*, const char*> names[] = {{"in_proj.weight", "in"}, {"conv.weight", "conv"}, {"conv.bias", "conv.b"},
                                                       {"dt_bias", "dt_bias"},   {"A_log", "A_log"},      {"D", "D"},
                                                       {"out_norm.weight", "norm"}, {"o_proj.weight", "o"}};
  for (const auto& n : names) ls.names[std::string("mixer.right.") + n.first] = p + "mix.right." + n.second;
  return make("state_space", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"value_dim", (double)vdim},
                              {"state_dim", (double)state}, {"groups", (double)groups}, {"norm_groups", (double)parts},
                              {"conv_taps", (double)taps}, {"eps", eps}});
}

ModelSpec povatar_model_spec(const Json& raw) {
  const int64_t width = positive(raw, "width", "the model's"), vocab = positive(raw, "vocab", "the model's");
  const double eps = finite(member(raw, "norm", "the model"), "eps", "norm");
  if (eps < 0) throw ConfigError("config.json: 'norm.eps' must not be negative");
  const double embed_scale = finite(member(raw, "embedding", "the model"), "scale", "embedding");
  const Json& layers = member(raw, "layers", "the model");
  if (layers.kind != Json::Array) throw ConfigError("config.json: 'layers' must be a list");
  const int64_t L = (int64_t)layers.items.size();
  const PartSpecPtr norm = make("rmsnorm", {{"size", (double)width}, {"eps", eps}});

  ModelSpec spec;
  spec.architecture = "Povatar";
  spec.vocab_size = vocab;
  spec.hidden_size = width;
  spec.max_positions = kMaxPositions;
  spec.embedding = make("token_embedding_scaled", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}, {"scale", embed_scale}});
  spec.final_norm = norm;
  spec.head = make("linear_head", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}});
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers.items[i];
    const std::string where = "layer " + std::to_string(i);
    const std::string p = "l" + std::to_string(i) + ".";
    const Json* type = l.get("type");
    if (!type || type->kind != Json::String) throw ConfigError("config.json: " + where + " lacks 'type'");
    if (type->text != "parallel") throw ConfigError("config.json: " + where + ": unknown mixer type '" + type->text + "'");
    const Json& m = member(l, "mixer", where);
    LayerSpec ls;
    ls.block = "parallel_sum";
    ls.block_numbers = {{"hidden_size", (double)width}};
    ls.norms = {{"mixer_in", norm}};
    ls.names = {{"norms.mixer_in.weight", p + "norm1"}, {"mixer.left_out", p + "mix.left.out"}, {"mixer.right_out", p + "mix.right.out"}};
    const PartSpecPtr left = left_mixer(member(m, "left", where + " mixer"), width, where + " left", p, ls);
    const PartSpecPtr right = right_mixer(member(m, "right", where + " mixer"), width, eps, where + " right", p, ls);
    ls.mixer = make("pair_mean", {{"hidden_size", (double)width}, {"eps", eps}}, {{"left_mixer", left}, {"right_mixer", right}});
    if (const Json* mlp = present(l, "mlp")) {
      const Json* kind = mlp->get("kind");
      if (!kind || kind->kind != Json::String || kind->text != "moe")
        throw ConfigError("config.json: " + where + ": the feed-forward's 'kind' must be 'moe'");
      const Json& router = member(*mlp, "router", where + " mlp");
      const int64_t experts = positive(router, "experts", where + " mlp.router"), top = positive(router, "top", where + " mlp.router");
      if (top > experts) throw ConfigError("config.json: " + where + ": 'top' must not exceed 'experts'");
      const int64_t ff = positive(member(*mlp, "expert", where + " mlp"), "ff", where + " mlp.expert");
      ls.feed_forward = make("routed_experts", {{"hidden_size", (double)width}, {"intermediate_size", (double)ff}, {"experts", (double)experts},
                                                {"top", (double)top}, {"weight_eps", kRouterWeightEps}});
      ls.norms["ffn_in"] = norm;
      ls.names["norms.ffn_in.weight"] = p + "norm2";
      ls.names["feed_forward.router.weight"] = p + "mlp.router";
      for (int64_t e = 0; e < experts; ++e) {
        const std::string n = std::to_string(e);
        ls.names["feed_forward.experts." + n + ".up_proj.weight"] = p + "mlp.e" + n + ".up";
        ls.names["feed_forward.experts." + n + ".down_proj.weight"] = p + "mlp.e" + n + ".down";
      }
    } else {
      ls.feed_forward = make("none", {});
      // The layer's second norm has nothing to feed; a checkpoint may still hold its weight.
      spec.ignored_names.push_back(p + "norm2");
    }
    spec.layers.push_back(std::move(ls));
    spec.schedule.push_back({(int)i, -1});
  }
  spec.names = {{"embedding.weight", "embed"}, {"final_norm.weight", "final.norm"}, {"head.weight", "head"}};
  spec.config_json = "{\"vocab\": " + std::to_string(vocab) + ", \"width\": " + std::to_string(width) + ", \"layers\": " + std::to_string(L) +
                     ", \"embedding_scale\": " + json_number(embed_scale) + ", \"norm_eps\": " + json_number(eps) + "}";
  return spec;
}

}  // namespace vosti
