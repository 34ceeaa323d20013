// The Miterax decoder: its config.json read and validated, and the model as data.
//
//   x = embed[token] + sinusoid(position)
//   layers in the order config "layers" lists them; config "loop" {start, stop, times} runs layers start .. stop-1
//   `times` times in a row with the same weights (each pass with a cache or state of its own) and adds row t of the
//   tensor "loop.step" to x before pass t
//   a layer:  h = norm1(x) (one learned gain);  x += ls1 * mixer(h) + ls2 * ff(h)
//   mixers:   "attention" (grouped queries, no rotation, query temperature, tanh-capped scores, softmax)
//             "mlstm"     (matrix memory with exponential gating)
//   ff:       dense, W_down xIELU(W_up h); a layer may have none
//   logits = head (final.norm(x))
//
// Keys: "width", "vocab", "norm": {"eps"}, "layers": [{"type", "mixer": {...}, "mlp": {"kind", "ff"} | null}],
// "loop": {"start", "stop", "times"} (optional).  Tensor names: "embed", "head", "final.norm", "loop.step",
// "l<i>.norm1", "l<i>.ls1", "l<i>.ls2", "l<i>.mix.*", "l<i>.mlp.*".
#include <cmath>

#include "../include/inference.h"

namespace tinyinfer {

namespace {
const Json& need(const Json& d, const char* key, const std::string& where) {
  const Json* v = d.find(key);
  if (!v || v->is_null()) throw ConfigError("config.json: " + where + "'" + key + "' is missing");
  return *v;
}
int64_t need_int(const Json& d, const char* key, const std::string& where, int64_t least = 1) {
  const Json& v = need(d, key, where);
  const bool whole = v.type() == Json::Int || (v.type() == Json::Float && v.as_double() == std::floor(v.as_double()));
  if (!whole) throw ConfigError("config.json: " + where + "'" + key + "' must be an integer, got " + v.dump());
  if (v.as_int() < least)
    throw ConfigError("config.json: " + where + "'" + key + "' must be at least " + std::to_string(least) + ", got " + v.dump());
  return v.as_int();
}
double need_float(const Json& d, const char* key, const std::string& where) {
  const Json& v = need(d, key, where);
  if (!v.is_number()) throw ConfigError("config.json: " + where + "'" + key + "' must be a number, got " + v.dump());
  return v.as_double();
}
bool given(const Json& d, const char* key) { return d.has(key); }
}  // namespace

// config.json with every default filled in; ConfigError names the key that is wrong
Json miterax_typed_config(const Json& d) {
  if (d.type() != Json::Object) throw ConfigError("config.json: top level must be a JSON object");
  Json out = Json::object();
  out.set("architecture", "Miterax");
  const int64_t width = need_int(d, "width", "");
  out.set("width", width);
  out.set("vocab", need_int(d, "vocab", ""));
  Json norm = Json::object();
  const double eps = need_float(need(d, "norm", ""), "eps", "norm: ");
  if (!(eps > 0.0)) throw ConfigError("config.json: norm: 'eps' must be positive");
  norm.set("eps", eps);
  out.set("norm", norm);
  const Json& layers = need(d, "layers", "");
  if (layers.type() != Json::Array || layers.size() == 0) throw ConfigError("config.json: 'layers' must be a list of at least one layer");
  Json ls = Json::array();
  for (size_t i = 0; i < layers.size(); ++i) {
    const std::string where = "layers[" + std::to_string(i) + "]: ";
    const Json& l = layers[i];
    if (l.type() != Json::Object) throw ConfigError("config.json: " + where + "must be an object");
    const Json& type = need(l, "type", where);
    const Json& m = need(l, "mixer", where);
    if (type.type() != Json::String || m.type() != Json::Object) throw ConfigError("config.json: " + where + "'type' must be a string and 'mixer' an object");
    Json lo = Json::object(), mo = Json::object();
    lo.set("type", type.as_string());
    const std::string mw = where + "mixer: ";
    const int64_t heads = need_int(m, "heads", mw);
    const int64_t dim = need_int(m, "dim", mw);
    mo.set("heads", heads);
    mo.set("dim", dim);
    mo.set("vdim", given(m, "vdim") ? need_int(m, "vdim", mw) : dim);
    if (type.as_string() == "attention") {
      const int64_t kv = given(m, "kv_heads") ? need_int(m, "kv_heads", mw) : heads;
      if (heads % kv) throw ConfigError("config.json: " + mw + "'heads' (" + std::to_string(heads) + ") must be a multiple of 'kv_heads' (" + std::to_string(kv) + ")");
      mo.set("kv_heads", kv);
      mo.set("scale", given(m, "scale") ? need_float(m, "scale", mw) : 1.0 / std::sqrt((double)dim));
      if (given(m, "softcap")) {
        const double cap = need_float(m, "softcap", mw);
        if (cap < 0.0) throw ConfigError("config.json: " + mw + "'softcap' must not be negative");
        mo.set("softcap", cap);
      } else {
        mo.set("softcap", Json());
      }
      if (given(m, "q_temp")) {
        Json qt = Json::object();
        qt.set("coef", need_float(m.at("q_temp"), "coef", mw + "q_temp: "));
        qt.set("every", need_int(m.at("q_temp"), "every", mw + "q_temp: "));
        mo.set("q_temp", qt);
      } else {
        mo.set("q_temp", Json());
      }
    } else if (type.as_string() == "mlstm") {
      const double cap = need_float(m, "gate_cap", mw);
      if (!(cap > 0.0)) throw ConfigError("config.json: " + mw + "'gate_cap' must be positive");
      mo.set("gate_cap", cap);
    } else {
      throw ConfigError("config.json: " + where + "'type' = '" + type.as_string() + "' is not served (attention, mlstm)");
    }
    lo.set("mixer", mo);
    const Json* mlp = l.find("mlp");
    if (mlp && !mlp->is_null()) {
      const std::string fw = where + "mlp: ";
      const std::string kind = given(*mlp, "kind") ? need(*mlp, "kind", fw).as_string() : "dense";
      if (kind != "dense") throw ConfigError("config.json: " + fw + "'kind' = '" + kind + "' is not served (dense)");
      Json fo = Json::object();
      fo.set("kind", kind);
      fo.set("ff", need_int(*mlp, "ff", fw));
      lo.set("mlp", fo);
    } else {
      lo.set("mlp", Json());
    }
    ls.push(lo);
  }
  out.set("layers", ls);
  const Json* loop = d.find("loop");
  if (loop && !loop->is_null()) {
    const int64_t L = (int64_t)layers.size();
    const int64_t start = need_int(*loop, "start", "loop: ", 0), stop = need_int(*loop, "stop", "loop: ", 0);
    const int64_t times = need_int(*loop, "times", "loop: ", 1);
    if (start > stop || stop > L)
      throw ConfigError("config.json: loop: 'start' " + std::to_string(start) + " and 'stop' " + std::to_string(stop) +
                        " must lie in order inside the " + std::to_string(L) + " layers");
    Json lo = Json::object();
    lo.set("start", start);
    lo.set("stop", stop);
    lo.set("times", times);
    out.set("loop", lo);
  } else {
    out.set("loop", Json());
  }
  return out;
}

ModelSpec miterax_spec(const Json& config) {
  const Json c = miterax_typed_config(config);
  const int64_t H = c.at("width").as_int(), V = c.at("vocab").as_int();
  const double eps = c.at("norm").at("eps").as_double();
  ModelSpec spec;
  spec.architecture = "Miterax";
  spec.vocab_size = V;
  spec.hidden_size = H;
  auto norm = [&](const std::string& tensor) {
    PartSpec p;
    p.kind = "rmsnorm";
    p.params.set("dim", H);
    p.params.set("eps", eps);
    p.params.set("scalar", true);
    p.params.set("tensor", tensor);
    return p;
  };
  spec.embedding.kind = "table";
  spec.embedding.params.set("vocab", V);
  spec.embedding.params.set("dim", H);
  spec.embedding.params.set("tensor", "embed");
  PartSpec pos;
  pos.kind = "sinusoidal";
  pos.params.set("dim", H);
  pos.params.set("base", 10000.0);
  spec.embedding.params.set("pos", pos.to_json());
  const Json& layers = c.at("layers");
  const int64_t L = (int64_t)layers.size();
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers[(size_t)i];
    const Json& m = l.at("mixer");
    LayerSpec ls;
    ls.prefix = "l" + std::to_string(i);
    ls.block.kind = "parallel";
    ls.block.params.set("dim", H);
    ls.block.params.set("scale1", "ls1");
    ls.block.params.set("scale2", "ls2");
    ls.parts.emplace_back("norm1", norm(ls.prefix + ".norm1"));
    PartSpec mix;
    mix.name = "mix";
    mix.params.set("hidden", H);
    mix.params.set("heads", m.at("heads").as_int());
    mix.params.set("head_dim", m.at("dim").as_int());
    mix.params.set("v_head_dim", m.at("vdim").as_int());
    if (l.at("type").as_string() == "attention") {
      mix.kind = "attention";
      mix.params.set("kv_heads", m.at("kv_heads").as_int());
      mix.params.set("qk_norm", false);
      mix.params.set("general", true);
      mix.params.set("scale", m.at("scale").as_double());
      if (m.has("softcap") && m.at("softcap").as_double() > 0.0) mix.params.set("softcap", m.at("softcap").as_double());
      if (m.has("q_temp")) mix.params.set("q_temp", m.at("q_temp"));
      for (const char* t : {"q", "k", "v", "o"}) mix.params.set(t, ls.prefix + ".mix." + t);
    } else {
      mix.kind = "mlstm";
      mix.params.set("gate_cap", m.at("gate_cap").as_double());
      mix.params.set("eps", eps);
    }
    ls.parts.emplace_back("mixer", mix);
    if (l.has("mlp")) {
      PartSpec ff;
      ff.kind = "dense";
      ff.name = "mlp";
      ff.params.set("hidden", H);
      ff.params.set("intermediate", l.at("mlp").at("ff").as_int());
      ff.params.set("activation", "xielu");
      ls.parts.emplace_back("ffn", ff);
    }
    spec.layers.push_back(std::move(ls));
  }
  // the loop: its passes are runs of the same layers; what is added before pass t is a layer of its own
  // (a row of "loop.step") in front of the pass
  if (c.has("loop")) {
    const Json& loop = c.at("loop");
    const int64_t start = loop.at("start").as_int(), stop = loop.at("stop").as_int(), times = loop.at("times").as_int();
    for (int64_t i = 0; i < start; ++i) spec.schedule.push_back((int)i);
    for (int64_t t = 0; t < times; ++t) {
      LayerSpec add;
      add.prefix = "";
      add.block.kind = "add_vector";
      add.block.params.set("dim", H);
      add.block.params.set("rows", times);
      add.block.params.set("row", t);
      add.block.params.set("tensor", "loop.step");
      spec.schedule.push_back((int)spec.layers.size());
      spec.layers.push_back(std::move(add));
      for (int64_t i = start; i < stop; ++i) spec.schedule.push_back((int)i);
    }
    for (int64_t i = stop; i < L; ++i) spec.schedule.push_back((int)i);
  }
  spec.final_norm = norm("final.norm");
  spec.lm_head.kind = "linear";
  spec.lm_head.params.set("vocab", V);
  spec.lm_head.params.set("dim", H);
  spec.lm_head.params.set("tied", false);
  spec.lm_head.params.set("tensor", "head");
  return spec;
}

}  // namespace tinyinfer
