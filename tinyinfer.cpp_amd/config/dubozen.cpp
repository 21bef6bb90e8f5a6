// The Dubozen decoder: its config.json read and validated, and the model as data.
//
//   x = LN(embed[token]) with the weight "embed.norm"; LN(z) = (z - mean) / sqrt(variance + eps) * w, no bias
//   the residual is kept in config "streams" copies x_1 .. x_S, all equal to x at the start.  Sublayer q of layer i (1: the
//   mixer, 2: the feed-forward) reads u = sum_s in[s] x_s through LN ("l<i>.norm<q>") and its output y goes back as
//   x_t <- sum_s mix[s, t] x_s + out[t] y with the tensors "l<i>.hc<q>.in / .out / .mix"; at the end x = sum_s x_s.
//   Without "streams" there is one x and x <- x + y.
//   mixers:  "attention"  grouped queries, a rotation of the first rot.dims entries of every head, scores (q . k) scale, causal,
//                         a learned sink a head in the softmax's denominator (".sink"); with "v_mix" the values of every such
//                         layer but the first are (1 - l) v + l v_first, l = ".vmix", v_first the first such layer's values of
//                         the same token; the heads' outputs times sigmoid(W_g h) entry by entry (".g"); W_o
//            "parallel"   left_scale * left + right_scale * right on the same input.  left (".left.*"): attention whose values
//                         are its keys as projected, RMS norms on every q and k head before the rotation (".q.norm", ".k.norm"),
//                         plain softmax, one gate number a head (".g" [heads, width]).  right (".right.*"): linear attention with
//                         a fixed decay per head on silu'd q, k, v, an RMS norm over all heads (".norm"), a sigmoid gate (".g")
//   ff:      "dense"      W_down (gelu_tanh(W_gate h) * (W_up h));  "moe": experts W_down (silu(W_gate h) * (W_up h)), sigmoid
//                         scores, ".correction" added for the choice only, groups.count groups of neighbours of which the
//                         groups.keep best (by the sum of their two largest choice scores) may be chosen from, weights
//                         s / (sum + 1e-20) * router.scale; a layer may have none
//   logits = embed LN(x) with the weight "final.norm"
//
// Keys: "width", "vocab", "norm": {"eps"}, "streams" (optional), "layers": [{"type", "mixer": {...}, "mlp": {...} | null}].
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

// "rot": {"base", "dims"} or absent; `most`: the entries a head has to turn
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
  return ro;
}

// what the softmax attention of either mixer gives: heads, kv_heads, dim, vdim, scale, rot
Json read_softmax_attention(const Json& m, const std::string& mw) {
  Json mo = Json::object();
  const int64_t heads = need_int(m, "heads", mw), dim = need_int(m, "dim", mw);
  const int64_t kv = given(m, "kv_heads") ? need_int(m, "kv_heads", mw) : heads;
  if (heads % kv) throw ConfigError("config.json: " + mw + "'heads' (" + std::to_string(heads) + ") must be a multiple of 'kv_heads' (" + std::to_string(kv) + ")");
  if (dim > 256) throw ConfigError("config.json: " + mw + "'dim' (" + std::to_string(dim) + ") is not served (up to 256)");
  mo.set("heads", heads);
  mo.set("kv_heads", kv);
  mo.set("dim", dim);
  mo.set("vdim", given(m, "vdim") ? need_int(m, "vdim", mw) : dim);
  if (mo.at("vdim").as_int() > 256) throw ConfigError("config.json: " + mw + "'vdim' is not served (up to 256)");
  mo.set("scale", given(m, "scale") ? need_float(m, "scale", mw) : 1.0 / std::sqrt((double)dim));
  mo.set("rot", read_rot(m, mw, dim));
  return mo;
}

PartSpec rotation(const Json& rot) {
  PartSpec pos;
  pos.kind = "rope_partial";
  pos.params.set("dims", rot.at("dims").as_int());
  pos.params.set("base", rot.at("base").as_double());
  return pos;
}
}  // namespace

// config.json with every default filled in; ConfigError names the key that is wrong
Json dubozen_typed_config(const Json& d) {
  if (d.type() != Json::Object) throw ConfigError("config.json: top level must be a JSON object");
  Json out = Json::object();
  out.set("architecture", "Dubozen");
  out.set("width", need_int(d, "width", ""));
  out.set("vocab", need_int(d, "vocab", ""));
  Json norm = Json::object();
  norm.set("eps", need_positive(need(d, "norm", ""), "eps", "norm: "));
  out.set("norm", norm);
  if (given(d, "streams")) {
    const int64_t streams = need_int(d, "streams", "");
    if (streams > 16) throw ConfigError("config.json: 'streams' (" + std::to_string(streams) + ") is not served (up to 16)");
    out.set("streams", streams);
  } else {
    out.set("streams", Json());
  }
  const Json& layers = need(d, "layers", "");
  if (layers.type() != Json::Array || layers.size() == 0) throw ConfigError("config.json: 'layers' must be a list of at least one layer");
  Json ls = Json::array();
  int64_t mixed_kv = 0, mixed_vdim = 0;
  for (size_t i = 0; i < layers.size(); ++i) {
    const std::string where = "layers[" + std::to_string(i) + "]: ";
    const Json& l = layers[i];
    if (l.type() != Json::Object) throw ConfigError("config.json: " + where + "must be an object");
    const Json& type = need(l, "type", where);
    const Json& m = need(l, "mixer", where);
    if (type.type() != Json::String || m.type() != Json::Object) throw ConfigError("config.json: " + where + "'type' must be a string and 'mixer' an object");
    Json lo = Json::object(), mo;
    lo.set("type", type.as_string());
    const std::string mw = where + "mixer: ";
    if (type.as_string() == "attention") {
      mo = read_softmax_attention(m, mw);
      const bool v_mix = given(m, "v_mix") && m.at("v_mix").type() == Json::Bool && m.at("v_mix").as_bool();
      if (given(m, "v_mix") && m.at("v_mix").type() != Json::Bool) throw ConfigError("config.json: " + mw + "'v_mix' must be true or false");
      mo.set("v_mix", v_mix);
      if (v_mix) {
        const int64_t kv = mo.at("kv_heads").as_int(), vdim = mo.at("vdim").as_int();
        if (mixed_kv && (mixed_kv != kv || mixed_vdim != vdim))
          throw ConfigError("config.json: " + mw + "layers that mix their values must agree in 'kv_heads' and 'vdim'");
        mixed_kv = kv;
        mixed_vdim = vdim;
      }
    } else if (type.as_string() == "parallel") {
      mo = Json::object();
      const Json& left = need(m, "left", mw);
      const Json& right = need(m, "right", mw);
      Json lm = read_softmax_attention(left, mw + "left: ");
      if (lm.at("vdim").as_int() != lm.at("dim").as_int())
        throw ConfigError("config.json: " + mw + "left: 'vdim' must equal 'dim' (the values are the keys)");
      mo.set("left", lm);
      const std::string rw = mw + "right: ";
      Json rm = Json::object();
      const int64_t heads = need_int(right, "heads", rw), dim = need_int(right, "dim", rw);
      const int64_t vdim = given(right, "vdim") ? need_int(right, "vdim", rw) : dim;
      if (dim > 256 || vdim > 256) throw ConfigError("config.json: " + rw + "'dim' and 'vdim' are served up to 256");
      rm.set("heads", heads);
      rm.set("dim", dim);
      rm.set("vdim", vdim);
      const Json& decay = need(right, "decay", rw);
      Json dl = Json::array();
      if (decay.is_number()) {      // one number: every head's
        for (int64_t j = 0; j < heads; ++j) dl.push(Json(decay.as_double()));
      } else {
        if (decay.type() != Json::Array || (int64_t)decay.size() != heads)
          throw ConfigError("config.json: " + rw + "'decay' must list one number a head (" + std::to_string(heads) + ")");
        for (const Json& v : decay.items()) {
          if (!v.is_number()) throw ConfigError("config.json: " + rw + "'decay' must hold numbers, got " + v.dump());
          dl.push(Json(v.as_double()));
        }
      }
      rm.set("decay", dl);
      mo.set("right", rm);
      mo.set("left_scale", given(m, "left_scale") ? need_float(m, "left_scale", mw) : 1.0);
      mo.set("right_scale", given(m, "right_scale") ? need_float(m, "right_scale", mw) : 1.0);
    } else {
      throw ConfigError("config.json: " + where + "'type' = '" + type.as_string() + "' is not served (attention, parallel)");
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
        Json eo = Json::object();
        eo.set("ff", need_int(need(*mlp, "expert", fw), "ff", fw + "expert: "));
        fo.set("expert", eo);
        const Json& router = need(*mlp, "router", fw);
        const std::string rw = fw + "router: ";
        const int64_t experts = need_int(router, "experts", rw), top = need_int(router, "top", rw);
        if (top > experts) throw ConfigError("config.json: " + rw + "'top' (" + std::to_string(top) + ") exceeds 'experts' (" + std::to_string(experts) + ")");
        Json ro = Json::object();
        ro.set("experts", experts);
        ro.set("top", top);
        ro.set("scale", given(router, "scale") ? need_float(router, "scale", rw) : 1.0);
        if (given(router, "groups")) {
          const Json& g = router.at("groups");
          const int64_t count = need_int(g, "count", rw + "groups: "), keep = need_int(g, "keep", rw + "groups: ");
          if (experts % count || keep > count || keep * (experts / count) < top)
            throw ConfigError("config.json: " + rw + "groups: " + std::to_string(count) + " groups of which " + std::to_string(keep) +
                              " are kept do not fit " + std::to_string(experts) + " experts and top " + std::to_string(top));
          Json go = Json::object();
          go.set("count", count);
          go.set("keep", keep);
          ro.set("groups", go);
        } else {
          ro.set("groups", Json());
        }
        fo.set("router", ro);
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
  return out;
}

ModelSpec dubozen_spec(const Json& config) {
  const Json c = dubozen_typed_config(config);
  const int64_t H = c.at("width").as_int(), V = c.at("vocab").as_int();
  const double eps = c.at("norm").at("eps").as_double();
  const int64_t S = c.has("streams") ? c.at("streams").as_int() : 0;
  ModelSpec spec;
  spec.architecture = "Dubozen";
  spec.vocab_size = V;
  spec.hidden_size = H;
  auto norm = [&](const std::string& tensor) {
    PartSpec p;
    p.kind = "layernorm";
    p.params.set("dim", H);
    p.params.set("eps", eps);
    p.params.set("tensor", tensor);
    return p;
  };
  // the softmax attention of either mixer, its tensors under `at`
  auto softmax_attention = [&](const Json& m, const std::string& at) {
    PartSpec mix;
    mix.kind = "attention";
    mix.params.set("hidden", H);
    mix.params.set("heads", m.at("heads").as_int());
    mix.params.set("kv_heads", m.at("kv_heads").as_int());
    mix.params.set("head_dim", m.at("dim").as_int());
    mix.params.set("v_head_dim", m.at("vdim").as_int());
    mix.params.set("scale", m.at("scale").as_double());
    mix.params.set("eps", eps);
    if (m.has("rot") && m.at("rot").at("dims").as_int() > 0) mix.params.set("pos", rotation(m.at("rot")).to_json());
    for (const char* t : {"q", "k", "v", "o"}) mix.params.set(t, at + "." + t);
    mix.params.set("gate_tensor", at + ".g");
    return mix;
  };
  spec.embedding.kind = "table";
  spec.embedding.params.set("vocab", V);
  spec.embedding.params.set("dim", H);
  spec.embedding.params.set("tensor", "embed");
  spec.embedding.params.set("norm", norm("embed.norm").to_json());
  const Json& layers = c.at("layers");
  const int64_t L = (int64_t)layers.size();
  bool first_mix_seen = false;
  for (int64_t i = 0; i < L; ++i) {
    const Json& l = layers[(size_t)i];
    const Json& m = l.at("mixer");
    LayerSpec ls;
    ls.prefix = "l" + std::to_string(i);
    ls.block.kind = S ? "hyper" : "pre_norm";
    if (S) {
      ls.block.params.set("streams", S);
      ls.block.params.set("dim", H);
      ls.block.params.set("defer_write", true);      // the block that sums the streams closes the run of layers
    }
    ls.parts.emplace_back("norm1", norm(ls.prefix + ".norm1"));
    const std::string at = ls.prefix + ".mix";
    PartSpec mix;
    if (l.at("type").as_string() == "attention") {
      mix = softmax_attention(m, at);
      mix.params.set("qk_norm", false);
      mix.params.set("sink", true);
      mix.params.set("sink_tensor", at + ".sink");
      mix.params.set("gate", "entry");
      mix.params.set("v_mix_tensor", at + ".vmix");
      if (m.at("v_mix").as_bool()) {
        mix.params.set("v_mix", first_mix_seen ? "mix" : "first");
        first_mix_seen = true;
      }
    } else {
      PartSpec left = softmax_attention(m.at("left"), at + ".left");
      left.name = "left";
      left.params.set("qk_norm", true);
      left.params.set("q_norm", at + ".left.q.norm");
      left.params.set("k_norm", at + ".left.k.norm");
      left.params.set("values_from_keys", true);
      left.params.set("gate", "head");
      const Json& r = m.at("right");
      PartSpec right;
      right.kind = "decay_attention";
      right.name = "right";
      right.params.set("hidden", H);
      right.params.set("heads", r.at("heads").as_int());
      right.params.set("head_dim", r.at("dim").as_int());
      right.params.set("v_head_dim", r.at("vdim").as_int());
      right.params.set("decay", r.at("decay"));
      right.params.set("eps", eps);
      mix.kind = "sum";
      mix.params.set("hidden", H);
      mix.params.set("left", left.to_json());
      mix.params.set("right", right.to_json());
      mix.params.set("left_scale", m.at("left_scale").as_double());
      mix.params.set("right_scale", m.at("right_scale").as_double());
    }
    mix.name = "mix";
    ls.parts.emplace_back("mixer", mix);
    if (l.has("mlp")) {
      const Json& f = l.at("mlp");
      ls.parts.emplace_back("norm2", norm(ls.prefix + ".norm2"));
      PartSpec ff;
      ff.name = "mlp";
      ff.params.set("hidden", H);
      if (f.at("kind").as_string() == "dense") {
        ff.kind = "glu";
        ff.params.set("intermediate", f.at("ff").as_int());
        ff.params.set("activation", "gelu_tanh");
      } else {
        const Json& r = f.at("router");
        ff.kind = "moe";
        ff.params.set("intermediate", f.at("expert").at("ff").as_int());
        ff.params.set("experts", r.at("experts").as_int());
        ff.params.set("top", r.at("top").as_int());
        ff.params.set("activation", "glu_silu");
        ff.params.set("score", "sigmoid");
        ff.params.set("renormalize", true);
        ff.params.set("sum_floor", 1e-20);
        ff.params.set("weight_scale", r.at("scale").as_double());
        ff.params.set("correction", true);
        if (r.has("groups")) ff.params.set("groups", r.at("groups"));
      }
      ls.parts.emplace_back("ffn", ff);
    }
    spec.layers.push_back(std::move(ls));
  }
  if (S) {
    // the streams are opened behind the embedding and closed in front of the final norm by layers of their own
    LayerSpec open, close;
    open.block.kind = "hyper_spread";
    close.block.kind = "hyper_sum";
    for (LayerSpec* b : {&open, &close}) {
      b->block.params.set("streams", S);
      b->block.params.set("dim", H);
    }
    spec.schedule.push_back((int)L);
    for (int64_t i = 0; i < L; ++i) spec.schedule.push_back((int)i);
    spec.schedule.push_back((int)L + 1);
    spec.layers.push_back(std::move(open));
    spec.layers.push_back(std::move(close));
  }
  spec.final_norm = norm("final.norm");
  spec.lm_head.kind = "linear";
  spec.lm_head.params.set("vocab", V);
  spec.lm_head.params.set("dim", H);
  spec.lm_head.params.set("tied", true);
  spec.lm_head.params.set("tied_to", "embed");
  return spec;
}

}  // namespace tinyinfer
