#include "tezinex.h"

#include <cmath>

namespace vosti {
namespace {

PartSpecPtr make(std::string kind, std::map<std::string, double> numbers) {
  auto p = std::make_shared<PartSpec>();
  p->kind = std::move(kind);
  p->numbers = std::move(numbers);
  return p;
}

const Json& member(const Json& j, const std::string& key, const std::string& where) {
  const Json* v = j.get(key);
  if (!v) throw ConfigError("config.json: " + where + " lacks '" + key + "'");
  return *v;
}

int64_t positive(const Json& j, const std::string& key, const std::string& where) {
  const Json& v = member(j, key, where);
  if (!v.is_int() || v.as_int() <= 0) throw ConfigError("config.json: " + where + " '" + key + "' must be a positive integer");
  return v.as_int();
}

int64_t not_negative(const Json& j, const std::string& key, const std::string& where) {
  const Json& v = member(j, key, where);
  if (!v.is_int() || v.as_int() < 0) throw ConfigError("config.json: " + where + " '" + key + "' must be an integer, zero or more");
  return v.as_int();
}

double finite(const Json& j, const std::string& key, const std::string& where) {
  const Json& v = member(j, key, where);
  if (v.kind != Json::Number || !std::isfinite(v.number)) throw ConfigError("config.json: " + where + " '" + key + "' must be a finite number");
  return v.number;
}

}  // namespace

// The constants that the design fixes stand here; everything else is read from the configuration.
constexpr double kSinusoidBase = 10000.0;   // the positions' angles are p * base^(-2i / width)
constexpr double kUnitNormEps = 1e-6;       // q and k of the delta rule: x / sqrt(sum(x^2) + this)
constexpr int64_t kMaxPositions = 1 << 22;  // the positions are computed, not tabulated; this bounds a request's length

ModelSpec tezinex_model_spec(const Json& raw) {
  const int64_t width = positive(raw, "width", "the model's"), vocab = positive(raw, "vocab", "the model's");
  if (width % 2) throw ConfigError("config.json: 'width' must be even for the sinusoidal positions");
  const double eps = finite(member(raw, "norm", "the model"), "eps", "norm");
  const double mult = finite(raw, "residual_mult", "the model's");
  const double logit_cap = raw.get("logit_softcap") ? finite(raw, "logit_softcap", "the model's") : 0.0;
  if (eps < 0 || logit_cap < 0) throw ConfigError("config.json: 'norm.eps' and 'logit_softcap' must not be negative");
  const Json& layers = member(raw, "layers", "the model");
  if (layers.kind != Json::Array) throw ConfigError("config.json: 'layers' must be a list");
  const int64_t L = (int64_t)layers.items.size();
  const PartSpecPtr norm = make("rmsnorm", {{"size", (double)width}, {"eps", eps}, {"offset", 1.0}});

  ModelSpec spec;
  spec.architecture = "Tezinex";
  spec.vocab_size = vocab;
  spec.hidden_size = width;
  spec.max_positions = kMaxPositions;
  spec.embedding = make("token_embedding_sinusoid", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}, {"base", kSinusoidBase}});
  spec.final_norm = norm;
  spec.head = make("linear_head", {{"vocab_size", (double)vocab}, {"hidden_size", (double)width}, {"tied", 1.0}, {"softcap", logit_cap}});
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers.items[i];
    const std::string where = "layer " + std::to_string(i);
    const std::string p = "l" + std::to_string(i) + ".";
    const Json* type = l.get("type");
    if (!type || type->kind != Json::String) throw ConfigError("config.json: " + where + " lacks 'type'");
    const Json& m = member(l, "mixer", where);
    LayerSpec ls;
    ls.block = "sandwich_depth";
    ls.block_numbers = {{"residual_mult", mult}, {"depth", (double)i}, {"states", (double)(L + 1)}, {"hidden_size", (double)width}};
    ls.names = {{"depth_weights", p + "dwa"}, {"norms.mixer_in.weight", p + "norm1"}, {"norms.mixer_out.weight", p + "norm1b"}};
    ls.norms = {{"mixer_in", norm}, {"mixer_out", norm}};
    int cache_from = -1;
    const int64_t heads = positive(m, "heads", where), kv_heads = positive(m, "kv_heads", where);
    const int64_t dim = positive(m, "dim", where), vdim = positive(m, "vdim", where);
    if (heads % kv_heads) throw ConfigError("config.json: " + where + ": 'heads' must be a multiple of 'kv_heads'");
    if (type->text == "attention") {
      const Json& mask = member(m, "mask", where);
      const int64_t window = positive(mask, "size", where + " mask"), keep = not_negative(mask, "keep_first", where + " mask");
      const double cap = m.get("softcap") ? finite(m, "softcap", where) : 0.0;
      const double scale = finite(m, "scale", where);
      if (scale <= 0 || cap < 0) throw ConfigError("config.json: " + where + ": 'scale' must be positive and 'softcap' not negative");
      if (const Json* from = m.get("kv_from")) {
        if (!from->is_int() || from->as_int() < 0 || from->as_int() >= i)
          throw ConfigError("config.json: " + where + ": 'kv_from' must name an earlier layer");
        cache_from = (int)from->as_int();
      }
      ls.mixer = make("attention", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"num_kv_heads", (double)kv_heads},
                                    {"head_dim", (double)dim}, {"value_dim", (double)vdim}, {"scale", scale}, {"window", (double)window},
                                    {"keep_first", (double)keep}, {"softcap", cap}, {"bias", 1.0}, {"sink", 1.0}, {"exact_weights", 1.0},
                                    {"own_kv", cache_from < 0 ? 1.0 : 0.0}});
      ls.names["mixer.q_proj.weight"] = p + "mix.q";
      ls.names["mixer.q_proj.bias"] = p + "mix.q.b";
      if (cache_from < 0) {
        ls.names["mixer.k_proj.weight"] = p + "mix.k";
        ls.names["mixer.k_proj.bias"] = p + "mix.k.b";
        ls.names["mixer.v_proj.weight"] = p + "mix.v";
        ls.names["mixer.v_proj.bias"] = p + "mix.v.b";
      }
      ls.names["mixer.sinks"] = p + "mix.sink";
      ls.names["mixer.o_proj.weight"] = p + "mix.o";
    } else if (type->text == "channel_delta") {
      const int64_t taps = positive(m, "conv", where);
      // The ranks of the two low-rank projections are not in the configuration: the tensors' shapes give them, and the
      // part reads them there (0 here).
      ls.mixer = make("channel_delta", {{"hidden_size", (double)width}, {"num_heads", (double)heads}, {"num_kv_heads", (double)kv_heads},
                                        {"key_dim", (double)dim}, {"value_dim", (double)vdim}, {"conv_taps", (double)taps}, {"eps", eps},
                                        {"unit_eps", kUnitNormEps}, {"decay_rank", 0.0}, {"gate_rank", 0.0}});
      const std::pair<const char*, const char*> names[] = {
          {"q_proj.weight", "q"},      {"q_conv.weight", "q.conv"},  {"k_proj.weight", "k"},         {"k_conv.weight", "k.conv"},
          {"v_proj.weight", "v"},      {"v_conv.weight", "v.conv"},  {"beta_proj.weight", "b"},      {"A_log", "A_log"},
          {"out_norm.weight", "norm"}, {"decay_down.weight", "a1"},  {"decay_up.weight", "a2"},      {"dt_bias", "dt_bias"},
          {"gate_down.weight", "g1"},  {"gate_up.weight", "g2"},     {"o_proj.weight", "o"}};
      for (const auto& n : names) ls.names[std::string("mixer.") + n.first] = p + "mix." + n.second;
    } else {
      throw ConfigError("config.json: " + where + ": unknown mixer type '" + type->text + "'");
    }
    if (const Json* mlp = l.get("mlp")) {
      const Json* kind = mlp->get("kind");
      if (!kind || kind->text != "dense") throw ConfigError("config.json: " + where + ": the feed-forward's 'kind' must be 'dense'");
      ls.feed_forward = make("swiglu", {{"hidden_size", (double)width}, {"intermediate_size", (double)positive(*mlp, "ff", where + " mlp")}});
      ls.norms["ffn_in"] = norm;
      ls.norms["ffn_out"] = norm;
      ls.names["norms.ffn_in.weight"] = p + "norm2";
      ls.names["norms.ffn_out.weight"] = p + "norm2b";
      for (const char* n : {"gate", "up", "down"}) ls.names[std::string("feed_forward.") + n + "_proj.weight"] = p + "mlp." + n;
    } else {
      ls.feed_forward = make("none", {});
    }
    spec.layers.push_back(std::move(ls));
    spec.schedule.push_back({(int)i, cache_from});
  }
  spec.names = {{"embedding.weight", "embed"}, {"final_norm.weight", "final.norm"}, {"head.weight", "embed"}};
  // The configuration is the typed one: it has no optional keys that a reader could resolve differently.
  std::string cfg = "{\"vocab\": " + std::to_string(vocab) + ", \"width\": " + std::to_string(width) + ", \"layers\": " + std::to_string(L) +
                    ", \"residual_mult\": " + json_number(mult) + ", \"norm_eps\": " + json_number(eps) + ", \"logit_softcap\": " +
                    json_number(logit_cap) + "}";
  spec.config_json = cfg;
  return spec;
}

}  // namespace vosti
