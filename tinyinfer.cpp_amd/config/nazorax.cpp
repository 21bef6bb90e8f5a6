// The Nazorax decoder: its config.json read and validated, and the model as data.
//
//   x = embed[token]; x0 = that embedding output
//   layers in the order config "layers" lists them; config "loop" {start, stop, times} runs layers start .. stop-1 `times`
//   times in a row with the same weights (each pass with a cache of its own), and right before the first layer of every
//   pass x <- W_in [x; x0] with the tensor "loop.in" [width, 2 width]
//   a layer:  h = norm1(x), Dynamic Tanh: tanh(alpha x) * w + b;  x += mixer(h) + ff(h)
//   mixers:   "attention"        grouped queries, biases on q, k, v, rotation of the first rot.dims entries of every head,
//                                a sliding window of mask.size positions, softmax
//             "latent_attention" a normed latent and one rotated key part per token, keys and values per head from the
//                                latent, YaRN-interpolated rotation, causal, a learned sink in the softmax's denominator
//   ff:       "dense" W_down (silu(W_gate h) * (W_up h)) with biases; "moe": experts with the clamped gated activation,
//             weights = softmax over the chosen logits, plus a shared expert; a layer may have none
//   logits = head final.norm(x)
//
// Keys: "width", "vocab", "norm": {"eps"}, "layers": [{"type", "mixer": {...}, "mlp": {...} | null}], "loop" (optional).
// Tensor names: "embed", "head", "final.norm{,.alpha,.b}", "loop.in", "l<i>.norm1{,.alpha,.b}", "l<i>.mix.*", "l<i>.mlp.*".
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

// "rot": {"base", "dims", "scaling": {factor, original, fast, slow} | absent}; `most`: the entries a head has to turn
Json read_rot(const Json& m, const std::string& mw, int64_t most) {
  if (!given(m, "rot")) return Json();
  const Json& r = m.at("rot");
  const std::string rw = mw + "rot: ";
  Json ro = Json::object();
  const int64_t dims = need_int(r, "dims", rw, 0);
  if (dims % 2 || dims > most)
    throw ConfigError("config.json: " + rw + "'dims' (" + std::to_string(dims) + ") must be even and at most " + std::to_string(most));
  ro.set("base", need_positive(r, "base", rw));
  ro.set("dims", dims);
  if (given(r, "scaling")) {
    Json so = Json::object();
    for (const char* key : {"factor", "original", "fast", "slow"}) so.set(key, need_positive(r.at("scaling"), key, rw + "scaling: "));
    ro.set("scaling", so);
  } else {
    ro.set("scaling", Json());
  }
  return ro;
}

// an expert's or the shared expert's sizes: {"ff", "limit"}
Json read_expert(const Json& e, const std::string& where) {
  Json o = Json::object();
  o.set("ff", need_int(e, "ff", where));
  o.set("limit", need_positive(e, "limit", where));
  return o;
}

PartSpec rotation(const Json& rot) {
  PartSpec pos;
  pos.kind = "rope_partial";
  pos.params.set("dims", rot.at("dims").as_int());
  pos.params.set("base", rot.at("base").as_double());
  if (rot.has("scaling")) pos.params.set("scaling", rot.at("scaling"));
  return pos;
}
}  // namespace

// config.json with every default filled in; ConfigError names the key that is wrong
Json nazorax_typed_config(const Json& d) {
  if (d.type() != Json::Object) throw ConfigError("config.json: top level must be a JSON object");
  Json out = Json::object();
  out.set("architecture", "Nazorax");
  out.set("width", need_int(d, "width", ""));
  out.set("vocab", need_int(d, "vocab", ""));
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
    Json lo = Json::object(), mo = Json::object();
    lo.set("type", type.as_string());
    const std::string mw = where + "mixer: ";
    const int64_t heads = need_int(m, "heads", mw);
    mo.set("heads", heads);
    if (type.as_string() == "attention") {
      const int64_t dim = need_int(m, "dim", mw);
      const int64_t kv = given(m, "kv_heads") ? need_int(m, "kv_heads", mw) : heads;
      if (heads % kv) throw ConfigError("config.json: " + mw + "'heads' (" + std::to_string(heads) + ") must be a multiple of 'kv_heads' (" + std::to_string(kv) + ")");
      mo.set("kv_heads", kv);
      mo.set("dim", dim);
      mo.set("vdim", given(m, "vdim") ? need_int(m, "vdim", mw) : dim);
      mo.set("scale", given(m, "scale") ? need_float(m, "scale", mw) : 1.0 / std::sqrt((double)dim));
      if (given(m, "mask")) {
        Json mask = Json::object();
        mask.set("size", need_int(m.at("mask"), "size", mw + "mask: "));
        mo.set("mask", mask);
      } else {
        mo.set("mask", Json());
      }
      mo.set("rot", read_rot(m, mw, dim));
    } else if (type.as_string() == "latent_attention") {
      const int64_t dim = need_int(m, "dim", mw), rot_dim = need_int(m, "rot_dim", mw, 0);
      mo.set("dim", dim);
      mo.set("rot_dim", rot_dim);
      mo.set("vdim", given(m, "vdim") ? need_int(m, "vdim", mw) : dim);
      mo.set("kv_rank", need_int(m, "kv_rank", mw));
      mo.set("scale", given(m, "scale") ? need_float(m, "scale", mw) : 1.0 / std::sqrt((double)(dim + rot_dim)));
      mo.set("rot", read_rot(m, mw, rot_dim));
    } else {
      throw ConfigError("config.json: " + where + "'type' = '" + type.as_string() + "' is not served (attention, latent_attention)");
    }
    lo.set("mixer", mo);
    const Json* mlp = l.find("mlp");
    if (mlp && !mlp->is_null()) {
      const std::string fw = where + "mlp: ";
      const std::string kind = given(*mlp, "kind") ? need(*mlp, "kind", fw).as_string() : "dense";
      Json fo = Json::object();
      fo.set("kind", kind);
      if (kind == "dense") {
        fo.set("ff", need_int(*mlp, "ff", fw));
      } else if (kind == "moe") {
        fo.set("expert", read_expert(need(*mlp, "expert", fw), fw + "expert: "));
        const Json& router = need(*mlp, "router", fw);
        const int64_t experts = need_int(router, "experts", fw + "router: "), top = need_int(router, "top", fw + "router: ");
        if (top > experts) throw ConfigError("config.json: " + fw + "router: 'top' (" + std::to_string(top) + ") exceeds 'experts' (" + std::to_string(experts) + ")");
        Json ro = Json::object();
        ro.set("experts", experts);
        ro.set("top", top);
        fo.set("router", ro);
        fo.set("shared", given(*mlp, "shared") ? read_expert(mlp->at("shared"), fw + "shared: ") : Json());
      } else {
        throw ConfigError("config.json: " + fw + "'kind' = '" + kind + "' is not served (dense, moe)");
      }
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
    if (start >= stop || stop > L)
      throw ConfigError("config.json: loop: 'start' " + std::to_string(start) + " must lie before 'stop' " + std::to_string(stop) +
                        ", both inside the " + std::to_string(L) + " layers");
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

ModelSpec nazorax_spec(const Json& config) {
  const Json c = nazorax_typed_config(config);
  const int64_t H = c.at("width").as_int(), V = c.at("vocab").as_int();
  const double eps = c.at("norm").at("eps").as_double();
  ModelSpec spec;
  spec.architecture = "Nazorax";
  spec.vocab_size = V;
  spec.hidden_size = H;
  auto norm = [&](const std::string& tensor) {
    PartSpec p;
    p.kind = "dyt";
    p.params.set("dim", H);
    p.params.set("tensor", tensor);
    return p;
  };
  auto expert = [&](const Json& e) {      // a gated feed-forward with the clamped activation, no biases
    PartSpec p;
    p.kind = "glu";
    p.params.set("hidden", H);
    p.params.set("intermediate", e.at("ff").as_int());
    p.params.set("activation", "clamped");
    p.params.set("limit", e.at("limit").as_double());
    return p;
  };
  spec.embedding.kind = "table";
  spec.embedding.params.set("vocab", V);
  spec.embedding.params.set("dim", H);
  spec.embedding.params.set("tensor", "embed");
  const Json& layers = c.at("layers");
  const int64_t L = (int64_t)layers.size();
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers[(size_t)i];
    const Json& m = l.at("mixer");
    LayerSpec ls;
    ls.prefix = "l" + std::to_string(i);
    ls.block.kind = "parallel";
    ls.block.params.set("dim", H);
    ls.parts.emplace_back("norm1", norm(ls.prefix + ".norm1"));
    PartSpec mix;
    mix.name = "mix";
    mix.params.set("hidden", H);
    mix.params.set("heads", m.at("heads").as_int());
    mix.params.set("head_dim", m.at("dim").as_int());
    mix.params.set("v_head_dim", m.at("vdim").as_int());
    mix.params.set("scale", m.at("scale").as_double());
    const bool turns = m.has("rot") && m.at("rot").at("dims").as_int() > 0;
    if (turns) mix.params.set("pos", rotation(m.at("rot")).to_json());
    if (l.at("type").as_string() == "attention") {
      mix.kind = "attention";
      mix.params.set("kv_heads", m.at("kv_heads").as_int());
      mix.params.set("qk_norm", false);
      mix.params.set("general", true);
      mix.params.set("bias", true);
      if (m.has("mask")) mix.params.set("window", m.at("mask").at("size").as_int());
      for (const char* t : {"q", "k", "v", "o"}) mix.params.set(t, ls.prefix + ".mix." + t);
    } else {
      mix.kind = "latent_attention";
      mix.params.set("rot_dim", m.at("rot_dim").as_int());
      mix.params.set("kv_rank", m.at("kv_rank").as_int());
      mix.params.set("eps", eps);
      mix.params.set("sink", true);
    }
    ls.parts.emplace_back("mixer", mix);
    if (l.has("mlp")) {
      const Json& f = l.at("mlp");
      PartSpec ff;
      ff.name = "mlp";
      ff.params.set("hidden", H);
      if (f.at("kind").as_string() == "dense") {
        ff.kind = "glu";
        ff.params.set("intermediate", f.at("ff").as_int());
        ff.params.set("activation", "silu");
        ff.params.set("bias", true);
      } else {
        ff.kind = "moe";
        ff.params.set("intermediate", f.at("expert").at("ff").as_int());
        ff.params.set("experts", f.at("router").at("experts").as_int());
        ff.params.set("top", f.at("router").at("top").as_int());
        ff.params.set("activation", "glu_clamped");
        ff.params.set("limit", f.at("expert").at("limit").as_double());
        ff.params.set("score", "softmax_chosen");
        ff.params.set("scale_input", false);
        if (f.has("shared")) {
          PartSpec sh = expert(f.at("shared"));
          sh.name = "shared";
          ff.params.set("shared", sh.to_json());
        }
      }
      ls.parts.emplace_back("ffn", ff);
    }
    spec.layers.push_back(std::move(ls));
  }
  // the loop: its passes are runs of the same layers; the embedding's output is kept right behind the embedding, and what
  // mixes it in again before a pass is a layer of its own in front of the pass
  if (c.has("loop")) {
    const Json& loop = c.at("loop");
    const int64_t start = loop.at("start").as_int(), stop = loop.at("stop").as_int(), times = loop.at("times").as_int();
    LayerSpec keep;
    keep.block.kind = "keep";
    keep.block.params.set("name", "embedding");
    spec.schedule.push_back((int)spec.layers.size());
    spec.layers.push_back(std::move(keep));
    LayerSpec mix;
    mix.block.kind = "mix_in";
    mix.block.params.set("dim", H);
    mix.block.params.set("from", "embedding");
    mix.block.params.set("tensor", "loop.in");
    const int mix_at = (int)spec.layers.size();
    spec.layers.push_back(std::move(mix));
    for (int64_t i = 0; i < start; ++i) spec.schedule.push_back((int)i);
    for (int64_t t = 0; t < times; ++t) {
      spec.schedule.push_back(mix_at);
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
