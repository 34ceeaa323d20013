// The Mumasun decoder: its config.json read and validated, and the model as data.
//
//   x = N(embed[token]), N the model's norm with the weight "embed.norm" (gain 1 + w)
//   layers in the order config "layers" lists them; a layer norms what a sublayer returns:
//     x += norm1(mixer(x));  x += norm2(ff(x))            (the sublayers read x itself; a layer may have no ff)
//   mixer "attention": differential attention (two softmax maps a head over one value, a1 - lambda a2, normed),
//     a short causal convolution behind the q, k and v projections, per-map RMS norm of q and k, rotation of the
//     first rot.dims entries with YaRN-interpolated frequencies, keys visible inside blocks of mask.size positions
//   ff "moe": experts W_down relu(W_up h)^2 chosen by sigmoid scores that multiply the experts' inputs
//   logits = embed final.norm(x) * logit_scale
//
// Keys: "width", "vocab", "logit_scale", "norm": {"eps"}, "layers": [{"type": "attention", "mixer": {"heads", "kv_heads",
// "dim", "vdim", "conv", "diff", "scale", "mask": {"size"}, "rot": {"base", "dims", "scaling": {"factor", "original",
// "fast", "slow"}}}, "mlp": {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}} | null}].
// Tensor names: "embed", "embed.norm", "final.norm", "l<i>.norm1", "l<i>.norm2", "l<i>.mix.{q,k,v,o}",
// "l<i>.mix.{q,k,v}.conv", "l<i>.mix.{q,k}.norm", "l<i>.mix.{lq1,lk1,lq2,lk2}", "l<i>.mlp.e<j>.{up,down}", "l<i>.mlp.router".
#include <cmath>

#include "../include/inference.h"

namespace tinyinfer {

namespace {
const Json& need(const Json& d, const char* key, const std::string& where) {
  const Json* v = d.type() == Json::Object ? d.find(key) : nullptr;
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
double need_positive(const Json& d, const char* key, const std::string& where) {
  const double v = need_float(d, key, where);
  if (!(v > 0.0)) throw ConfigError("config.json: " + where + "'" + key + "' must be positive");
  return v;
}
bool given(const Json& d, const char* key) { return d.type() == Json::Object && d.has(key); }
}  // namespace

// config.json with every default filled in; ConfigError names the key that is wrong
Json mumasun_typed_config(const Json& d) {
  if (d.type() != Json::Object) throw ConfigError("config.json: top level must be a JSON object");
  Json out = Json::object();
  out.set("architecture", "Mumasun");
  out.set("width", need_int(d, "width", ""));
  out.set("vocab", need_int(d, "vocab", ""));
  out.set("logit_scale", given(d, "logit_scale") ? need_float(d, "logit_scale", "") : 1.0);
  Json norm = Json::object();
  norm.set("eps", need_positive(need(d, "norm", ""), "eps", "norm: "));
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
    if (type.as_string() != "attention")
      throw ConfigError("config.json: " + where + "'type' = '" + type.as_string() + "' is not served (attention)");
    Json lo = Json::object(), mo = Json::object();
    lo.set("type", type.as_string());
    const std::string mw = where + "mixer: ";
    const int64_t heads = need_int(m, "heads", mw), dim = need_int(m, "dim", mw);
    const int64_t kv = given(m, "kv_heads") ? need_int(m, "kv_heads", mw) : heads;
    if (heads % kv) throw ConfigError("config.json: " + mw + "'heads' (" + std::to_string(heads) + ") must be a multiple of 'kv_heads' (" + std::to_string(kv) + ")");
    mo.set("heads", heads);
    mo.set("kv_heads", kv);
    mo.set("dim", dim);
    mo.set("vdim", given(m, "vdim") ? need_int(m, "vdim", mw) : dim);
    mo.set("conv", given(m, "conv") ? Json(need_int(m, "conv", mw)) : Json());      // one tap: a factor per channel
    mo.set("diff", need_float(m, "diff", mw));
    mo.set("scale", given(m, "scale") ? need_float(m, "scale", mw) : 1.0 / std::sqrt((double)dim));
    if (given(m, "mask")) {
      Json mask = Json::object();
      mask.set("size", need_int(m.at("mask"), "size", mw + "mask: "));
      mo.set("mask", mask);
    } else {
      mo.set("mask", Json());
    }
    if (given(m, "rot")) {
      const Json& r = m.at("rot");
      const std::string rw = mw + "rot: ";
      Json ro = Json::object();
      const int64_t dims = need_int(r, "dims", rw, 0);
      if (dims % 2 || dims > dim) throw ConfigError("config.json: " + rw + "'dims' (" + std::to_string(dims) + ") must be even and at most 'dim'");
      ro.set("base", need_positive(r, "base", rw));
      ro.set("dims", dims);
      if (given(r, "scaling")) {
        Json so = Json::object();
        for (const char* key : {"factor", "original", "fast", "slow"}) so.set(key, need_positive(r.at("scaling"), key, rw + "scaling: "));
        ro.set("scaling", so);
      } else {
        ro.set("scaling", Json());
      }
      mo.set("rot", ro);
    } else {
      mo.set("rot", Json());
    }
    lo.set("mixer", mo);
    const Json* mlp = l.find("mlp");
    if (mlp && !mlp->is_null()) {
      const std::string fw = where + "mlp: ";
      const std::string kind = given(*mlp, "kind") ? need(*mlp, "kind", fw).as_string() : "moe";
      if (kind != "moe") throw ConfigError("config.json: " + fw + "'kind' = '" + kind + "' is not served (moe)");
      Json fo = Json::object(), eo = Json::object(), ro = Json::object();
      fo.set("kind", kind);
      eo.set("ff", need_int(need(*mlp, "expert", fw), "ff", fw + "expert: "));
      const Json& router = need(*mlp, "router", fw);
      const int64_t experts = need_int(router, "experts", fw + "router: "), top = need_int(router, "top", fw + "router: ");
      if (top > experts) throw ConfigError("config.json: " + fw + "router: 'top' (" + std::to_string(top) + ") exceeds 'experts' (" + std::to_string(experts) + ")");
      ro.set("experts", experts);
      ro.set("top", top);
      fo.set("expert", eo);
      fo.set("router", ro);
      lo.set("mlp", fo);
    } else {
      lo.set("mlp", Json());
    }
    ls.push(lo);
  }
  out.set("layers", ls);
  return out;
}

ModelSpec mumasun_spec(const Json& config) {
  const Json c = mumasun_typed_config(config);
  const int64_t H = c.at("width").as_int(), V = c.at("vocab").as_int();
  const double eps = c.at("norm").at("eps").as_double();
  ModelSpec spec;
  spec.architecture = "Mumasun";
  spec.vocab_size = V;
  spec.hidden_size = H;
  auto norm = [&](const std::string& tensor) {
    PartSpec p;
    p.kind = "rmsnorm";
    p.params.set("dim", H);
    p.params.set("eps", eps);
    p.params.set("one_plus", true);
    p.params.set("tensor", tensor);
    return p;
  };
  spec.embedding.kind = "table";
  spec.embedding.params.set("vocab", V);
  spec.embedding.params.set("dim", H);
  spec.embedding.params.set("tensor", "embed");
  spec.embedding.params.set("norm", norm("embed.norm").to_json());
  const Json& layers = c.at("layers");
  for (size_t i = 0; i < layers.size(); ++i) {
    const Json& l = layers[i];
    const Json& m = l.at("mixer");
    LayerSpec ls;
    ls.prefix = "l" + std::to_string(i);
    ls.block.kind = "post_norm";
    ls.parts.emplace_back("norm1", norm(ls.prefix + ".norm1"));
    PartSpec mix;
    mix.kind = "diff_attention";
    mix.name = "mix";
    const int64_t heads = m.at("heads").as_int(), kv = m.at("kv_heads").as_int(), dim = m.at("dim").as_int(), vdim = m.at("vdim").as_int();
    mix.params.set("hidden", H);
    mix.params.set("heads", heads);
    mix.params.set("kv_heads", kv);
    mix.params.set("head_dim", dim);
    mix.params.set("v_head_dim", vdim);
    mix.params.set("diff", m.at("diff").as_double());
    mix.params.set("scale", m.at("scale").as_double());
    mix.params.set("eps", eps);
    if (m.has("mask")) mix.params.set("block", m.at("mask").at("size").as_int());
    if (m.has("rot") && m.at("rot").at("dims").as_int() > 0) {
      PartSpec pos;
      pos.kind = "rope_partial";
      pos.params.set("dims", m.at("rot").at("dims").as_int());
      pos.params.set("base", m.at("rot").at("base").as_double());
      if (m.at("rot").has("scaling")) pos.params.set("scaling", m.at("rot").at("scaling"));
      mix.params.set("pos", pos.to_json());
    }
    if (m.has("conv")) {
      const std::string base = ls.prefix + ".mix.";
      PartSpec conv;
      conv.kind = "short_conv";
      conv.params.set("taps", m.at("conv").as_int());
      Json segments = Json::array();
      const std::pair<const char*, int64_t> runs[3] = {{"q", heads * 2 * dim}, {"k", kv * 2 * dim}, {"v", kv * vdim}};
      for (const auto& r : runs) {
        Json s = Json::array();
        s.push(base + r.first + ".conv");
        s.push(r.second);
        segments.push(s);
      }
      conv.params.set("segments", segments);
      mix.params.set("conv", conv.to_json());
    }
    ls.parts.emplace_back("mixer", mix);
    if (l.has("mlp")) {
      const Json& f = l.at("mlp");
      PartSpec ff;
      ff.kind = "moe";
      ff.name = "mlp";
      ff.params.set("hidden", H);
      ff.params.set("intermediate", f.at("expert").at("ff").as_int());
      ff.params.set("experts", f.at("router").at("experts").as_int());
      ff.params.set("top", f.at("router").at("top").as_int());
      ff.params.set("activation", "relu2");
      ff.params.set("score", "sigmoid");
      ff.params.set("renormalize", false);
      ff.params.set("scale_input", true);
      ls.parts.emplace_back("norm2", norm(ls.prefix + ".norm2"));
      ls.parts.emplace_back("ffn", ff);
    }
    spec.layers.push_back(std::move(ls));
  }
  spec.final_norm = norm("final.norm");
  spec.lm_head.kind = "linear";
  spec.lm_head.params.set("vocab", V);
  spec.lm_head.params.set("dim", H);
  spec.lm_head.params.set("tied", true);
  spec.lm_head.params.set("tied_to", "embed");
  spec.lm_head.params.set("scale", c.at("logit_scale").as_double());
  return spec;
}

}  // namespace tinyinfer
