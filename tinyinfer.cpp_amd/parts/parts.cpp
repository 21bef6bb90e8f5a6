// The parts a model is put together from, and their registry by family and kind.
//
//   embedding "table"     x[m, :] = float(E[tok[m], :]), no scaling (/root/reference/src/inference.cu:14-24)
//   norm      "rmsnorm"   y = x * rsqrt(mean(x^2) + eps) * w, eps inside the root, the weight multiplies
//                         directly (/root/reference/src/cuda/rms_norm.cu:15-25)
//   pos       "rope_neox" half-split rotation over the whole head: pair (k, k + hd/2) turns by
//                         pos * theta^(-2k/hd) (/root/reference/src/cuda/attention.cu:38,64-74; the
//                         adjacent-pair variant is the mistake listed in docs/report.md:91)
//   mixer     "attention" causal grouped-query attention over the paged cache: fused q/k/v product, per-head
//                         RMSNorm of q and k with a weight shared by all heads (before rotation; v is left
//                         alone), rotation, cache write, head h reads kv head h / (heads / kv_heads), scores
//                         scaled by 1/sqrt(hd), output projection added into the residual
//                         (/root/reference/src/inference.cu:41-55; src/cuda/attention.cu:12-87,107-198)
//   ffn       "swiglu"    y = silu(h Wg^T) * (h Wu^T); x += y Wd^T, gate and up rows held as one matrix
//                         (/root/reference/src/inference.cu:60-65,155-160; src/cuda/ffn.cu:13-15)
//   block     "pre_norm"  x += mixer(norm1(x)); x += ffn(norm2(x)) (/root/reference/src/inference.cu:35-66)
//   head      "linear"    logits = h E_out^T with E_out the embedding itself or a matrix of its own
//                         (/root/reference/src/cuda/lm_head.cu:5-10; the reference is always tied, src/model.h:42)
//
//
// Parts no layer of the reference has (their formulas stand at each class):
//   pos       "sinusoidal"  a vector of sines and cosines of the position added to the residual behind the embedding
//   norm      "rmsnorm" with `scalar`: one learned number as the gain of every channel
//   mixer     "attention" with `v_head_dim`, `softcap`, `q_temp`: keys and values of different sizes, tanh-capped
//                           scores, a query factor that grows with the logarithm of the position
//   mixer     "mlstm"       the mLSTM cell: a matrix memory per head, kept as per-request state
//   ffn       "dense"       down(act(up h)) with the xIELU activation
//   block     "parallel"    x += s1 * mixer(norm(x)) + s2 * ffn(norm(x)) with learned per-channel scales
//   block     "add_vector"  x += a row of a learned table (what a looped run of layers adds before each pass)
//
//   norm      "rmsnorm" with `one_plus`: the checkpoint holds the gain minus one; the norm onto the residual (forward_add)
//   embedding "table" with `norm`: a norm of the looked-up rows, in 32-bit, in place
//   pos       "rope_partial" rotation of the first `dims` entries of a head, frequencies interpolated between the plain
//                           ones and the ones divided by `factor` (YaRN), cosine and sine times 0.1 ln(factor) + 1
//   filter    "short_conv"  a causal convolution of a few taps over time on every channel, the last taps - 1 rows as state
//   mixer     "diff_attention" two softmax maps a head over one value, subtracted, normed; keys visible per block
//   ffn       "moe"         routed experts with sigmoid or softmax scores on the experts' inputs or outputs
//   block     "post_norm"   x += norm1(mixer(x)); x += norm2(ffn(x)): the sublayers read x itself
//
//
//   norm      "dyt"         Dynamic Tanh: tanh(alpha x) * w + b with one learned number alpha; no mean, no variance
//   mixer     "attention" with `bias` (biases on q, k, v) and a `pos` beside keys and values of their own sizes
//   mixer     "latent_attention" a token keeps one normed latent and one rotated key part; keys and values per head come from
//                           the latent; a learned sink in the softmax's denominator
//   ffn       "glu"         down(act(gate h, up h)) with act silu(g) u or the clamped g sigmoid(alpha g) (u + 1); optional biases
//   ffn       "moe" with `activation` "glu_clamped", `score` "softmax_chosen" and a `shared` feed-forward every token takes
//   block     "keep"        keeps a copy of the residual under a name for a later block of the step
//   block     "mix_in"      x <- W [x; kept]: the residual and a kept stream through one learned matrix
//
//
//   norm      "layernorm"   (x - mean) / sqrt(variance + eps) * w: a gain, no bias; also of a weighted sum of several streams
//   block     "hyper"       the residual in several streams (hyper-connections): a sublayer reads norm(sum_s a_s x_s) and its output
//                           y goes back as x_t <- sum_s B[s, t] x_s + c_t y; "hyper_spread" / "hyper_sum" open and close the streams
//   mixer     "attention" with `sink` (a learned number a head in the softmax's denominator), `gate` (a sigmoid gate on the
//                           heads' outputs, "entry" or "head"), `values_from_keys`, `v_mix` (values mixed with the first such
//                           layer's), and a per-head norm beside keys and values of their own sizes
//   mixer     "decay_attention" linear attention with a fixed decay per head, its state per request
//   mixer     "sum"         two mixers side by side on the same input, added with fixed factors
//   ffn       "glu" with `activation` "gelu_tanh"; "moe" with `correction`, `groups`, `weight_scale`, `sum_floor`
//
// A part gets every size and constant as a parameter and never looks at the model it sits in.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <mutex>

#include "../include/inference.h"

namespace tinyinfer {

std::vector<std::string> Part::child_slots() const {
  std::vector<std::string> names;
  const size_t n = children().size();
  for (size_t i = 0; i < n; ++i) names.push_back(std::to_string(i));
  return names;
}

void Part::walk(const std::function<void(Part&)>& fn) {
  fn(*this);
  for (const auto& c : children()) c->walk(fn);
}

static std::string join(const std::string& prefix, const std::string& name) {
  if (prefix.empty()) return name;
  if (name.empty()) return prefix;
  return prefix + "." + name;
}

// ----------------------------------------------------------------------------------- registry
namespace {
struct Registered {
  PartFactory factory;
  std::vector<std::pair<std::string, std::string>> slots;
};
std::mutex g_parts_mutex;
std::map<std::pair<std::string, std::string>, Registered>& table() {
  static std::map<std::pair<std::string, std::string>, Registered> t;
  return t;
}
const char* FAMILIES[] = {"embedding", "norm", "pos", "mixer", "ffn", "block", "head", "filter"};
void register_builtin_parts();
void ensure_builtins() {
  static std::once_flag once;
  std::call_once(once, register_builtin_parts);
}
int64_t param_int(const Json& p, const char* key) {
  const Json* v = p.find(key);
  if (!v || !v->is_number()) throw ConfigError(std::string("part parameter '") + key + "' is missing or not a number");
  return v->as_int();
}
double param_float(const Json& p, const char* key) {
  const Json* v = p.find(key);
  if (!v || !v->is_number()) throw ConfigError(std::string("part parameter '") + key + "' is missing or not a number");
  return v->as_double();
}
// a tensor's name in the checkpoint: the parameter `key` gives it in full, else prefix + "." + fallback
std::string tensor_name(const Json& p, const char* key, const std::string& prefix, const char* fallback) {
  const Json* v = p.find(key);
  if (v && v->type() == Json::String) return v->as_string();
  if (prefix.empty()) return fallback;
  return prefix + "." + fallback;
}
}  // namespace

void NormPart::forward_add(StepContext&, const Tensor&, const Tensor&, bool, const int*, int, const Tensor*) {
  throw EngineError(std::string("the norm '") + kind_name() + "' cannot write into the residual");
}
Rows NormPart::forward_mixed(StepContext&, const Tensor&, const Tensor&) {
  throw EngineError(std::string("the norm '") + kind_name() + "' has no form for a sum of streams");
}
void MixerPart::forward_pair(StepContext&, const Rows&, const Tensor&, const Tensor&, float&, float&) {
  throw EngineError(std::string("the mixer '") + kind_name() + "' does not leave its output as a pair");
}
void MixerPart::forward_store(StepContext&, const Rows&, const Tensor&) {
  throw EngineError(std::string("the mixer '") + kind_name() + "' cannot write its output apart from the residual");
}
void FeedForwardPart::forward_store(StepContext&, const Rows&, const Tensor&) {
  throw EngineError(std::string("the feed-forward '") + kind_name() + "' cannot write its output apart from the residual");
}

void register_part(const std::string& family, const std::string& kind, PartFactory factory,
                   std::vector<std::pair<std::string, std::string>> slots) {
  bool ok = false;
  for (const char* f : FAMILIES) ok = ok || family == f;
  if (!ok) throw ConfigError("unknown part family '" + family + "'");
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  table()[{family, kind}] = Registered{std::move(factory), std::move(slots)};
}

bool part_registered(const std::string& family, const std::string& kind) {
  ensure_builtins();
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  return table().count({family, kind}) != 0;
}

std::vector<std::string> registered_parts(const std::string& family) {
  ensure_builtins();
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  std::vector<std::string> kinds;
  for (const auto& kv : table())
    if (kv.first.first == family) kinds.push_back(kv.first.second);
  return kinds;
}

std::vector<std::pair<std::string, std::string>> block_slots(const std::string& kind) {
  ensure_builtins();
  std::lock_guard<std::mutex> lock(g_parts_mutex);
  auto it = table().find({"block", kind});
  if (it == table().end()) throw ConfigError("no block arrangement of kind '" + kind + "'");
  return it->second.slots;
}

std::shared_ptr<Part> build_part(const std::string& family, const PartSpec& spec, const std::string& prefix,
                                 const PartChildren& children) {
  ensure_builtins();
  PartFactory factory;
  {
    std::lock_guard<std::mutex> lock(g_parts_mutex);
    auto it = table().find({family, spec.kind});
    if (it == table().end()) {
      std::string have;
      for (const auto& kv : table())
        if (kv.first.first == family) have += (have.empty() ? "'" : ", '") + kv.first.second + "'";
      throw ConfigError("no " + family + " part of kind '" + spec.kind + "'; registered: [" + have + "]");
    }
    factory = it->second.factory;
  }
  std::shared_ptr<Part> part = factory(prefix, spec.params, children);
  if (!part) throw ConfigError("the factory of " + family + " '" + spec.kind + "' returned no part");
  if (family != part->family())
    throw ConfigError("the factory of " + family + " '" + spec.kind + "' returned a part of family '" + part->family() + "'");
  if (part->built_kind.empty()) {
    part->built_kind = spec.kind;
    part->built_from = spec.params;
  }
  return part;
}

// ------------------------------------------------------------------------------- built-in parts
namespace {

// `tensor`: the table's name in the checkpoint (default: prefix + ".weight").  `pos`: an additive position
// encoding (a part of family "pos" with additive() true), added to every row behind the lookup.
class Embedding final : public EmbeddingPart {
 public:
  Embedding(const std::string& prefix, const Json& p, const PartChildren& children)
      : EmbeddingPart(prefix), vocab(param_int(p, "vocab")), dim(param_int(p, "dim")), name(tensor_name(p, "tensor", prefix, "weight")) {
    for (const auto& c : children)
      if (c.first == "pos") pos = std::dynamic_pointer_cast<PositionPart>(c.second);
    if (!pos && p.has("pos")) pos = std::dynamic_pointer_cast<PositionPart>(build_part("pos", PartSpec::from_json(p.at("pos")), prefix));
    if (pos && !pos->additive()) throw ConfigError("embedding: the position encoding '" + std::string(pos->kind_name()) + "' is not additive");
    for (const auto& c : children)
      if (c.first == "norm") norm = std::dynamic_pointer_cast<NormPart>(c.second);
    if (!norm && p.has("norm")) norm = std::dynamic_pointer_cast<NormPart>(build_part("norm", PartSpec::from_json(p.at("norm")), prefix));
    if (norm && !norm->can_add()) throw ConfigError("embedding: the norm '" + std::string(norm->kind_name()) + "' cannot write 32-bit rows");
  }
  const char* kind_name() const override { return "table"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    n.shape = {vocab, dim};
    return {{name, n}};
  }
  std::vector<std::shared_ptr<Part>> children() const override {
    std::vector<std::shared_ptr<Part>> v;
    if (pos) v.push_back(pos);
    if (norm) v.push_back(norm);
    return v;
  }
  std::vector<std::string> child_slots() const override {
    std::vector<std::string> v;
    if (pos) v.push_back("pos");
    if (norm) v.push_back("norm");
    return v;
  }
  void load(WeightSource& src) override { weight = src.fetch(name, tensors()[0].second); }
  void forward(StepContext& ctx, const Tensor& x) override {
    ctx.ops.embed(weight, ctx.tokens, ctx.M, x, ctx.fed_tokens, ctx.n_fed_tokens);
    if (pos) pos->add(ctx, x);
    if (norm) norm->forward_add(ctx, x, x, false);
  }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t vocab, dim;
  std::string name;
  std::shared_ptr<PositionPart> pos;
  std::shared_ptr<NormPart> norm;      // `norm`: applied to the looked-up rows (after `pos`), in 32-bit
  Tensor weight;
};

// `scale`: the logits are multiplied by it.
// `tied`: 1 reads `tied_to`; 0 reads its own `weight`; -1 takes its own weight if the checkpoint
// holds one and `tied_to` otherwise.
class LMHead final : public HeadPart {
 public:
  LMHead(const std::string& prefix, int64_t vocab, int64_t dim, int tied, std::string tied_to, std::string own_name, double scale = 1.0)
      : HeadPart(prefix), vocab(vocab), dim(dim), tied(tied), tied_to(std::move(tied_to)), own_name(std::move(own_name)), scale((float)scale) {}
  const char* kind_name() const override { return "linear"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed must, may;
    must.shape = may.shape = {vocab, dim};
    may.optional = true;
    const std::string& own = own_name;
    if (tied == 0) return {{own, must}};
    // a checkpoint that still carries the duplicate is accepted
    return {{tied_to, must}, {own, may}};
  }
  void load(WeightSource& src) override {
    const std::string& own = own_name;
    TensorNeed n;
    n.shape = {vocab, dim};
    if (tied == 0 || (tied < 0 && src.has(own))) weight = src.fetch(own, n);
    else weight = src.fetch(tied_to, n);      // the source hands out one copy per name: the embedding's
  }
  Tensor forward(StepContext& ctx, const Rows& h) override {
    const Tensor& rows = h.materialize(ctx.ops);
    Tensor logits = ctx.buf("head.logits", DType::F32, {rows.shape[0], vocab});
    ctx.ops.linear(rows, weight, logits, Ops::Store);
    if (scale != 1.f) ctx.ops.scale(logits, scale);
    return logits;
  }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t vocab, dim;
  int tied;
  std::string tied_to, own_name;
  float scale;                 // `scale`: a factor on the logits
  Tensor weight;
};

// `scalar`: the checkpoint holds one number, the gain of every channel (y = x / rms(x) * g); it is spread
// over a vector when the weights load, so every kernel that takes a norm's weight serves it.  `tensor`:
// the weight's name in the checkpoint (default: prefix + ".weight").
class RMSNorm final : public NormPart {
 public:
  RMSNorm(const std::string& prefix, int64_t dim, double eps, bool scalar = false, std::string name_ = "", bool one_plus = false)
      : NormPart(prefix), dim(dim), eps((float)eps), scalar(scalar), one_plus(one_plus),
        name(name_.empty() ? join(prefix, "weight") : std::move(name_)) {}
  const char* kind_name() const override { return "rmsnorm"; }
  bool can_be_lazy() const override { return true; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    if (!scalar) n.shape = {dim};
    n.role = TensorNeed::Vector;
    n.a = one_plus ? 0.0 : 1.0;
    n.b = 0.1;
    return {{name, n}};
  }
  void load(WeightSource& src) override {
    if (one_plus) {
      // the gain is 1 + w, formed once in 32-bit (the stored tensor may serve another part as it is)
      const Tensor stored = src.fetch(name, tensors()[0].second);
      if (scalar) {
        const Tensor one = src.alloc(DType::F32, {1});
        plus_one(stored, one, src.to_host);
        weight = src.alloc(DType::F32, {dim});
        spread(one, weight, src.to_host);
      } else {
        weight = src.alloc(DType::F32, {dim});
        plus_one(stored, weight, src.to_host);
      }
      return;
    }
    if (!scalar) {
      weight = src.fetch(name, tensors()[0].second);
      return;
    }
    const Tensor one = src.fetch(name, tensors()[0].second);
    weight = src.alloc(DType::F32, {dim});
    spread(one, weight, src.to_host);
  }
  static void spread(const Tensor& one, const Tensor& all, bool on_host);     // all[:] = one[0]
  static void plus_one(const Tensor& w, const Tensor& out, bool on_host);     // out = 1 + w
  bool can_add() const override { return true; }
  void forward_add(StepContext& ctx, const Tensor& y, const Tensor& x, bool accumulate, const int* gather, int n_gather,
                   const Tensor* rounded) override {
    ctx.ops.norm_residual(x, y, weight, eps, accumulate, gather, n_gather, rounded);
  }
  // x: f32 [M, dim].  With `rows` only those rows of x are read, in that order.  `lazy`: the
  // consumer feeds the result to one product and nothing else, so where a kernel can take the
  // norm in, the rows come back not yet computed.
  Rows forward(StepContext& ctx, const Tensor& x, const int* rows, int64_t n_rows, bool lazy) override {
    const int64_t n = rows ? n_rows : x.shape[0];
    Rows r;
    r.t = ctx.buf("norm.out", ctx.act_dtype, {n, dim});
    if (lazy && !rows && ctx.ops.can_fuse_norm(n, r.t.dtype)) {
      r.lazy = true;
      r.x = x;
      r.weight = weight;
      r.eps = eps;
      return r;
    }
    ctx.ops.rmsnorm(x, weight, eps, r.t, rows, n_rows);
    return r;
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t dim;
  float eps;
  bool scalar, one_plus;     // one_plus: the checkpoint holds the gain minus one (weights kept around zero)
  std::string name;
  Tensor weight;
};

// An additive position encoding: entry 2i of a position's vector is sin(p * base^(-2i / dim)), entry 2i + 1 the
// cosine of the same angle.  The frequencies are built on the host in double precision and rounded to 32-bit;
// the angle and its sine and cosine are 32-bit on the device.
class Sinusoidal final : public PositionPart {
 public:
  Sinusoidal(const std::string& prefix, int64_t dim, double base) : PositionPart(prefix), dim(dim), base(base) {
    if (dim <= 0 || !(base > 0.0)) throw ConfigError("sinusoidal positions: dim and base must be positive");
  }
  const char* kind_name() const override { return "sinusoidal"; }
  bool additive() const override { return true; }
  bool reads_through_ops() const override { return true; }
  void prepare(Ops&, int) override {
    if (inv_freq.data()) return;
    const int64_t half = (dim + 1) / 2;
    std::vector<float> host((size_t)half);
    for (int64_t i = 0; i < half; ++i) host[(size_t)i] = (float)std::pow(base, -2.0 * (double)i / (double)dim);
    inv_freq = DeviceBuffer((size_t)half * 4);
    upload(inv_freq.data(), host.data(), (size_t)half * 4);
  }
  void add(StepContext& ctx, const Tensor& x) override {
    prepare(ctx.ops, 0);
    ctx.ops.add_sinusoid(x, ctx.positions, Tensor(inv_freq.data(), DType::F32, {(dim + 1) / 2}));
  }
  void apply(StepContext&, const Tensor&, const Tensor&) override {
    throw EngineError("sinusoidal positions are added to the residual; they do not rotate queries and keys");
  }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    if (!inv_freq.data()) return {};
    return {{"inv_freq", Tensor(inv_freq.data(), DType::F32, {(dim + 1) / 2})}};
  }
  static void upload(void* dst, const void* src, size_t bytes);
  int64_t dim;
  double base;
  DeviceBuffer inv_freq;
};

// The inverse frequencies are built once on the host in double precision and rounded to float.
// `prepare(n)` tabulates cosine and sine for positions below n, on the host, from the angle in double
// precision (rounded to float only at the end): a 32-bit angle pos * inv_freq[k] is pos * 2^-23 off, 6e-4
// five thousand tokens in, and differently at every position, so that not only distances would count.
// Positions beyond the table (none that an engine serves) have the angle and its sine and cosine in
// 32-bit on the device, as /root/reference/src/cuda/rope.cu:20-22 has them everywhere.
//
// A table never changes and is never freed while anything may read it: captured graphs hold its
// address in their kernel arguments.  Parts with the same head size and base share the longest table
// made so far; an engine that needs a longer one makes a new table, and every part keeps each table
// it has ever handed out until the part itself goes (its model outlives the engines on it).
struct RopeTable {
  int head_dim = 0;
  double theta = 0;
  DeviceBuffer inv_freq, table;
  int table_len = 0;
};
std::mutex g_rope_mutex;
std::map<std::pair<int, double>, std::weak_ptr<RopeTable>>& rope_tables() {
  static std::map<std::pair<int, double>, std::weak_ptr<RopeTable>> m;
  return m;
}

class RotaryNeox final : public PositionPart {
 public:
  RotaryNeox(const std::string& prefix, int64_t head_dim, double theta) : PositionPart(prefix), head_dim((int)head_dim), theta(theta) {
    if (head_dim % 2) throw ConfigError("rotary: head_dim " + std::to_string(head_dim) + " must be even");
  }
  const char* kind_name() const override { return "rope_neox"; }
  // the table this part reads now (null before the first use)
  std::shared_ptr<RopeTable> current() const {
    std::lock_guard<std::mutex> lock(g_rope_mutex);
    return kept.empty() ? nullptr : kept.back();
  }
  // a table of at least `len` positions (0: the frequencies alone will do)
  std::shared_ptr<RopeTable> table_for(int len) {
    std::lock_guard<std::mutex> lock(g_rope_mutex);
    if (!kept.empty() && kept.back()->table_len >= len) return kept.back();
    auto& slot = rope_tables()[{head_dim, theta}];
    std::shared_ptr<RopeTable> t = slot.lock();
    if (!t || t->table_len < len) {
      t = std::make_shared<RopeTable>();
      t->head_dim = head_dim;
      t->theta = theta;
      const int half = head_dim / 2;
      std::vector<double> inv(half);
      std::vector<float> inv32(half);
      for (int k = 0; k < half; ++k) {
        inv[k] = std::pow(theta, -2.0 * k / head_dim);
        inv32[k] = (float)inv[k];
      }
      t->inv_freq = DeviceBuffer((size_t)half * 4);
      upload(t->inv_freq.data(), inv32.data(), (size_t)half * 4);
      if (len > 0) {
        std::vector<float> host((size_t)len * half * 2);
        for (int p = 0; p < len; ++p)
          for (int k = 0; k < half; ++k) {
            const double angle = (double)p * inv[k];
            host[((size_t)p * half + k) * 2] = (float)std::cos(angle);
            host[((size_t)p * half + k) * 2 + 1] = (float)std::sin(angle);
          }
        t->table = DeviceBuffer(host.size() * 4);
        upload(t->table.data(), host.data(), host.size() * 4);
        t->table_len = len;
      }
      slot = t;
    }
    kept.push_back(t);
    return t;
  }
  void prepare(Ops&, int max_seq) override { table_for(max_seq); }
  bool fused(Ops::Rotation& rot) const override {
    const std::shared_ptr<RopeTable> t = current();
    if (!t) return false;
    rot.inv_freq = (const float*)t->inv_freq.data();
    rot.table = (const float*)t->table.data();
    rot.table_len = t->table_len;
    return true;
  }
  void apply(StepContext& ctx, const Tensor& q, const Tensor& k) override {
    const Tensor inv = inv_freq_tensor(ctx.ops);
    ctx.ops.rope_neox(q, ctx.positions, inv);
    if (k.defined()) ctx.ops.rope_neox(k, ctx.positions, inv);
  }
  Tensor inv_freq_tensor(Ops&) { return Tensor(table_for(0)->inv_freq.data(), DType::F32, {head_dim / 2}); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    const std::shared_ptr<RopeTable> t = current();
    if (!t) return {};
    const int half = head_dim / 2;
    std::vector<std::pair<std::string, Tensor>> h = {{"inv_freq", Tensor(t->inv_freq.data(), DType::F32, {half})}};
    if (t->table_len) h.emplace_back("table", Tensor(t->table.data(), DType::F32, {t->table_len, half, 2}));
    return h;
  }
  static void upload(void* dst, const void* src, size_t bytes);
  int head_dim;
  double theta;
  std::vector<std::shared_ptr<RopeTable>> kept;     // oldest first; the last one is read
};

class SwiGLU final : public FeedForwardPart {
 public:
  SwiGLU(const std::string& prefix, int64_t hidden, int64_t intermediate)
      : FeedForwardPart(prefix), hidden(hidden), intermediate(intermediate) {}
  const char* kind_name() const override { return "swiglu"; }
  bool takes_lazy_norm() const override { return true; }      // h goes into one product and nowhere else
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed up, down;
    up.shape = {intermediate, hidden};
    down.shape = {hidden, intermediate};
    return {{join(prefix, "gate_proj.weight"), up}, {join(prefix, "up_proj.weight"), up},
            {join(prefix, "down_proj.weight"), down}};
  }
  void load(WeightSource& src) override {
    // gate and up go straight into one matrix [2F, H]: one product yields both
    w_gate_up = src.alloc(src.matrix_dtype, {2 * intermediate, hidden});
    src.fill(join(prefix, "gate_proj.weight"), w_gate_up.rows(0, intermediate));
    src.fill(join(prefix, "up_proj.weight"), w_gate_up.rows(intermediate, intermediate));
    w_down = src.alloc(src.matrix_dtype, {hidden, intermediate});
    src.fill(join(prefix, "down_proj.weight"), w_down);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor y = ctx.buf("ffn.y", ctx.act_dtype, {h.t.shape[0], intermediate});
    ctx.ops.linear(h, w_gate_up, y, Ops::SwiGLU);
    ctx.ops.linear(y, w_down, x, Ops::Add, /*may_defer=*/true);
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w_gate_up", w_gate_up}, {"w_down", w_down}}; }
  int64_t hidden, intermediate;
  Tensor w_gate_up, w_down;
};

const int PREFILL_TILE_Q = 128;      // query rows per work item of the tiled attention kernels
const int PREFILL_TILE_SMALL = 64;   // and of the kernel that pairs a tile of many keys with one of few

class Attention final : public MixerPart {
 public:
  Attention(const std::string& prefix, const Json& p, const PartChildren& children) : MixerPart(prefix) {
    hidden = param_int(p, "hidden");
    heads = (int)param_int(p, "heads");
    kv_heads = (int)param_int(p, "kv_heads");
    head_dim = (int)param_int(p, "head_dim");
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
      throw ConfigError("attention: heads " + std::to_string(heads) + " not a multiple of kv_heads " + std::to_string(kv_heads));
    v_dim = p.has("v_head_dim") ? (int)param_int(p, "v_head_dim") : head_dim;
    softcap = p.has("softcap") ? (float)param_float(p, "softcap") : 0.f;
    if (p.has("q_temp")) {
      const Json& qt = p.at("q_temp");
      temp_coef = (float)param_float(qt, "coef");
      temp_every = (int)param_int(qt, "every");
      if (temp_every <= 0) throw ConfigError("attention: q_temp.every must be positive");
    }
    qk_norm = p.has("qk_norm") ? p.at("qk_norm").as_bool() : true;
    // capped scores, a query temperature or values of another size than the keys: the kernels that serve these take
    // any sizes up to 256 and neither a per-head norm nor a rotation
    bias = p.has("bias") && p.at("bias").as_bool();
    // a sink, a gate, values from the keys or mixed with another layer's: the gated kernels (any sizes up to 256, a per-head norm too)
    has_sink = p.has("sink") && p.at("sink").as_bool();
    if (p.has("gate")) {
      const std::string g = p.at("gate").as_string();
      if (g != "entry" && g != "head") throw ConfigError("attention: gate '" + g + "' is not served (entry, head)");
      gate_mode = g == "entry" ? 1 : 2;
    }
    values_from_keys = p.has("values_from_keys") && p.at("values_from_keys").as_bool();
    if (p.has("v_mix")) {
      const std::string vm = p.at("v_mix").as_string();
      if (vm != "first" && vm != "mix") throw ConfigError("attention: v_mix '" + vm + "' is not served (first, mix)");
      mix_mode = vm == "first" ? 1 : 2;
    }
    gated = has_sink || gate_mode != 0 || values_from_keys || mix_mode != 0;
    if (gated) {
      if (softcap > 0.f || temp_coef != 0.f || bias || (p.has("shares_kv") && p.at("shares_kv").as_bool()))
        throw ConfigError("attention: a sink, a gate, values from the keys or mixed values go with neither capped scores, a query "
                          "temperature, biases nor a shared cache");
      if (values_from_keys && v_dim != head_dim) throw ConfigError("attention: values that are the keys have the keys' size");
      if (values_from_keys && mix_mode) throw ConfigError("attention: values that are the keys are not mixed");
    }
    general = gated || softcap > 0.f || temp_coef != 0.f || v_dim != head_dim || bias || (p.has("general") && p.at("general").as_bool());
    if (gated) {
      if (head_dim < 1 || head_dim > 256 || v_dim < 1 || v_dim > 256)
        throw ConfigError("attention: key size " + std::to_string(head_dim) + " / value size " + std::to_string(v_dim) +
                          " are not served (up to 256)");
    } else if (general) {
      if (head_dim < 1 || head_dim > 256 || v_dim < 1 || v_dim > 256)
        throw ConfigError("attention: key size " + std::to_string(head_dim) + " / value size " + std::to_string(v_dim) +
                          " are not served (up to 256)");
      if (qk_norm || (p.has("shares_kv") && p.at("shares_kv").as_bool()))
        throw ConfigError("attention: capped scores, a query temperature, biases or a separate value size go with neither a per-head norm "
                          "nor a shared cache");
    } else if (head_dim < 16 || head_dim % 16 || head_dim > 256) {
      // every other attention kernel's range (float32 and bfloat16 alike): refused when the part is built, not at its first step
      throw ConfigError("attention: head_dim " + std::to_string(head_dim) +
                        " is not served: the attention kernels take head sizes in steps of 16 up to 256");
    }
    eps = (float)(p.has("eps") ? p.at("eps").as_double() : 1e-6);
    window = p.has("window") ? (int)p.at("window").as_int() : 0;
    scale = p.has("scale") ? (float)p.at("scale").as_double() : (float)(1.0 / std::sqrt((double)head_dim));
    shares_kv = p.has("shares_kv") && p.at("shares_kv").as_bool();
    for (const auto& c : children)
      if (c.first == "pos") pos = std::dynamic_pointer_cast<PositionPart>(c.second);
    if (!pos && p.has("pos")) pos = std::dynamic_pointer_cast<PositionPart>(build_part("pos", PartSpec::from_json(p.at("pos")), prefix));
    nq = (int64_t)heads * head_dim;
    nk = shares_kv ? 0 : (int64_t)kv_heads * head_dim;
    nv = shares_kv || values_from_keys ? 0 : (int64_t)kv_heads * v_dim;
    no = (int64_t)heads * v_dim;
    ng = gate_mode == 1 ? no : gate_mode == 2 ? heads : 0;
    n_qn = tensor_name(p, "q_norm", prefix, "q_norm.weight");
    n_kn = tensor_name(p, "k_norm", prefix, "k_norm.weight");
    n_sink = tensor_name(p, "sink_tensor", prefix, "sink");
    n_gate = tensor_name(p, "gate_tensor", prefix, "g");
    n_vmix = tensor_name(p, "v_mix_tensor", prefix, "vmix");
    vmix_named = p.has("v_mix_tensor");
    n_q = tensor_name(p, "q", prefix, "q_proj.weight");
    n_k = tensor_name(p, "k", prefix, "k_proj.weight");
    n_v = tensor_name(p, "v", prefix, "v_proj.weight");
    n_o = tensor_name(p, "o", prefix, "o_proj.weight");
  }
  const char* kind_name() const override { return "attention"; }
  bool can_store() const override { return general; }
  bool takes_lazy_norm() const override { return true; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    if (pos) return {pos};
    return {};
  }
  std::vector<std::string> child_slots() const override {
    if (pos) return {"pos"};
    return {};
  }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    TensorNeed q, kv, vv, o, nw;
    q.shape = {nq, hidden};
    kv.shape = {nk, hidden};
    vv.shape = {nv, hidden};
    o.shape = {hidden, no};
    nw.shape = {head_dim};
    nw.role = TensorNeed::Vector;
    nw.a = 1.0;
    nw.b = 0.1;
    t.emplace_back(n_q, q);
    t.emplace_back(n_o, o);
    if (!shares_kv) {
      t.emplace_back(n_k, kv);
      if (!values_from_keys) t.emplace_back(n_v, vv);
    }
    if (qk_norm) {
      t.emplace_back(n_qn, nw);
      if (!shares_kv) t.emplace_back(n_kn, nw);
    }
    if (has_sink) {
      TensorNeed sk;
      sk.shape = {(int64_t)heads};
      sk.role = TensorNeed::Vector;
      sk.b = 1.0;
      t.emplace_back(n_sink, sk);
    }
    if (gate_mode) {
      TensorNeed g;
      g.shape = {ng, hidden};
      t.emplace_back(n_gate, g);
    }
    if (mix_mode || vmix_named) {      // one number; the layer whose values the others mix in holds it too, unused; a layer that
      TensorNeed lam;                  // mixes nothing accepts one the checkpoint may carry
      lam.optional = mix_mode == 0;
      lam.role = TensorNeed::Vector;
      lam.init = "uniform";
      lam.a = 0.2;
      lam.b = 0.6;
      t.emplace_back(n_vmix, lam);
    }
    if (bias) {
      // the biases of the projections: the tensor's name with ".b"
      const std::pair<const std::string*, int64_t> runs[3] = {{&n_q, nq}, {&n_k, nk}, {&n_v, nv}};
      for (const auto& r : runs) {
        TensorNeed b;
        b.shape = {r.second};
        b.role = TensorNeed::Vector;
        b.b = 0.3;
        t.emplace_back(*r.first + ".b", b);
      }
    }
    return t;
  }
  void load(WeightSource& src) override {
    if (bias) {
      b_qkv = src.alloc(DType::F32, {nq + nk + nv});
      src.fill(n_q + ".b", b_qkv.rows(0, nq));
      src.fill(n_k + ".b", b_qkv.rows(nq, nk));
      src.fill(n_v + ".b", b_qkv.rows(nq + nk, nv));
    }
    // q, k and v go straight into the fused matrix (the reference builds its fused copy beside the
    // originals and keeps both: /root/reference/src/inference.cu:154-169)
    w_qkv = src.alloc(src.matrix_dtype, {nq + nk + nv + ng, hidden});      // the gate's rows behind q, k and v: one product
    src.fill(n_q, w_qkv.rows(0, nq));
    if (!shares_kv) {
      src.fill(n_k, w_qkv.rows(nq, nk));
      if (nv) src.fill(n_v, w_qkv.rows(nq + nk, nv));
    }
    if (ng) src.fill(n_gate, w_qkv.rows(nq + nk + nv, ng));
    w_o = src.alloc(src.matrix_dtype, {hidden, no});
    src.fill(n_o, w_o);
    if (qk_norm) {
      TensorNeed nw;
      nw.shape = {head_dim};
      nw.role = TensorNeed::Vector;
      q_norm_w = src.fetch(n_qn, nw);
      if (!shares_kv) k_norm_w = src.fetch(n_kn, nw);
    }
    for (const auto& kv : tensors()) {
      if (has_sink && kv.first == n_sink) sink = src.fetch(kv.first, kv.second);
      if (mix_mode && kv.first == n_vmix) mix_lambda = src.fetch(kv.first, kv.second);
    }
  }
  bool has_cache() const override { return true; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::PagedKV;
    n.kv_heads = kv_heads;
    n.head_dim = head_dim;
    // gated layers whose values are smaller than keys of a size the matrix cores take: the pages hold the values padded with
    // zeros to the keys' size, so that the kernels that hold keys and values of one size read them
    const bool padded = gated && v_dim < head_dim && (head_dim == 32 || head_dim == 64 || head_dim == 128);
    n.v_dim = (v_dim != head_dim && !padded) ? v_dim : 0;
    n.window = window;
    return n;
  }

  // The work lists of the attention kernels for this step: query tiles of 128 rows in order,
  // tiles of 64 rows from the one whose last row sees the most keys to the one that sees the
  // fewest, and the rows of single-token entries.  Every attention part of a model asks for the
  // same lists; the first one builds them.
  void plan(StepPlan& plan) const override {
    if (plan.decode_only() || plan.has("attention.tiles")) return;
    const auto& entries = plan.entries();
    size_t n_tiles = 0, n_small = 0, n_dec = 0;
    for (const auto& e : entries) {
      if (e.n_tokens > 1) {
        n_tiles += (e.n_tokens + PREFILL_TILE_Q - 1) / PREFILL_TILE_Q;
        n_small += (e.n_tokens + PREFILL_TILE_SMALL - 1) / PREFILL_TILE_SMALL;
      } else {
        ++n_dec;
      }
    }
    int* tiles = plan.ints("attention.tiles", 2 * n_tiles);
    int* small = plan.ints("attention.tiles_small", 2 * n_small);
    int* dec = plan.ints("attention.decode_rows", n_dec);
    struct Small { int last, entry, row; };
    std::vector<Small> order;
    order.reserve(n_small);
    int portion_context = 0;
    size_t t = 0, d = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
      const auto& e = entries[i];
      if (e.n_tokens > 1) {
        for (int q0 = 0; q0 < e.n_tokens; q0 += PREFILL_TILE_Q) {
          tiles[t++] = (int)i;
          tiles[t++] = e.row0 + q0;
        }
        for (int q0 = 0; q0 < e.n_tokens; q0 += PREFILL_TILE_SMALL)
          order.push_back({e.start + std::min(q0 + PREFILL_TILE_SMALL, e.n_tokens) - 1, (int)i, e.row0 + q0});
        portion_context = std::max(portion_context, e.start + e.n_tokens);
      } else {
        dec[d++] = e.row0;
      }
    }
    std::stable_sort(order.begin(), order.end(), [](const Small& a, const Small& b) { return a.last > b.last; });
    for (size_t i = 0; i < order.size(); ++i) {
      small[2 * i] = order[i].entry;
      small[2 * i + 1] = order[i].row;
    }
    plan.set_value("attention.portion_context", portion_context);
  }

  AttentionWork work(const StepContext& ctx) const {
    AttentionWork w;
    w.M = ctx.M;
    w.positions = ctx.positions;
    w.slots = ctx.slots;
    w.entry_meta = ctx.entry_meta;
    w.decode_only = ctx.decode_only;
    w.slots_are_rows = ctx.decode_only;      // every entry is one row: a row's entry is the row itself
    w.max_context = ctx.max_context;
    w.split_context = ctx.max_context;
    if (!ctx.decode_only) {
      w.tiles = ctx.planned("attention.tiles");
      w.n_tiles = (int)(ctx.planned_size("attention.tiles") / 2);
      w.tiles_small = ctx.planned("attention.tiles_small");
      w.n_tiles_small = (int)(ctx.planned_size("attention.tiles_small") / 2);
      w.decode_rows = ctx.planned("attention.decode_rows");
      w.n_decode_rows = (int)ctx.planned_size("attention.decode_rows");
      w.portion_context = (int)ctx.value("attention.portion_context");
    }
    if (ctx.plan && ctx.plan->sized_for_longest()) {
      // a graph is being captured: what a replay launches must cover the longest sequence
      w.split_context = ctx.plan->max_seq();
      if (w.n_tiles) w.portion_context = std::max(w.portion_context, ctx.plan->max_seq() / 2);
    }
    return w;
  }

  // Capped scores, a query temperature, values of their own size: the projections in 32-bit, q times its temperature
  // and k, v into the pages, attention with scores, cap and softmax in 32-bit, then the output projection.
  void run_general(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor qkv = ctx.buf("attn.qkv", DType::F32, {M, nq + nk + nv});
    ctx.ops.linear(h, w_qkv, qkv, Ops::Store);
    const auto bound = ctx.binding(this);
    const Tensor pool = ctx.kv_pool(bound.first, bound.second);
    const Ops::CacheView view = ctx.cache_view(bound.first);
    Tensor q = ctx.buf("attn.q", ctx.act_dtype, {M, nq});
    Ops::Rotation rot;
    if (pos && !pos->fused(rot)) throw EngineError("attention: the position encoding '" + std::string(pos->kind_name()) + "' has no fused form");
    if (bias || pos)
      ctx.ops.qkv_split_write(qkv, b_qkv, rot, ctx.positions, ctx.slots, view, pool, q, heads, kv_heads, head_dim, v_dim, temp_coef, temp_every);
    else
      ctx.ops.qkv_split_write(qkv, ctx.positions, ctx.slots, view, pool, q, heads, kv_heads, head_dim, v_dim, temp_coef, temp_every);
    Tensor a = ctx.buf("attn.out", ctx.act_dtype, {M, no});
    if (v_dim == head_dim && head_dim % 16 == 0)      // the step's tiles through the matrix cores where they serve the size, else row by row
      ctx.ops.attention(work(ctx), ctx.ws, view, q, pool, a, heads, kv_heads, head_dim, scale, window, softcap);
    else
      ctx.ops.attention_capped(q, pool, view, ctx.positions, ctx.slots, a, heads, kv_heads, head_dim, v_dim, scale, softcap, window);
    ctx.ops.linear(a, w_o, out, epi, epi == Ops::Add);
  }
  // A sink, a gate, values from the keys or mixed with the first such layer's: one product with the stacked weight
  // [q; k; v; gate] (32-bit sums), the preparation (per-head norms, rotation, the values' mixing, q out, k and v into the
  // pages), attention with the sink in the denominator and the gate on its output, then the output projection.
  void run_gated(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor proj = ctx.buf("attn.qkv", DType::F32, {M, nq + nk + nv + ng});
    ctx.ops.linear(h, w_qkv, proj, Ops::Store);
    const auto bound = ctx.binding(this);
    const Tensor pool = ctx.kv_pool(bound.first, bound.second);
    const Ops::CacheView view = ctx.cache_view(bound.first);
    Tensor q = ctx.buf("attn.q", ctx.act_dtype, {M, nq});
    Ops::Rotation rot;
    if (pos && !pos->fused(rot)) throw EngineError("attention: the position encoding '" + std::string(pos->kind_name()) + "' has no fused form");
    Ops::QkvColumns cols;
    cols.q = 0;
    cols.k = (int)nq;
    cols.v = values_from_keys ? -1 : (int)(nq + nk);
    Ops::ValueMix mix;
    mix.mode = mix_mode;
    if (mix_mode) {
      mix.kept = ctx.buf("attn.v_kept", DType::F32, {M, nv});
      mix.lambda = mix_lambda;
    }
    ctx.ops.gated_qkv_prep(proj, cols, q_norm_w, k_norm_w, eps, rot, mix, ctx.positions, ctx.slots, view, pool, q, heads, kv_heads,
                           head_dim, v_dim);
    Tensor a = ctx.buf("attn.out", ctx.act_dtype, {M, no});
    Ops::AttentionGate gate;
    gate.mode = gate_mode;
    gate.proj = proj;
    gate.col = (int)(nq + nk + nv);
    const AttentionWork w = work(ctx);
    ctx.ops.gated_attention(q, pool, view, ctx.positions, ctx.slots, sink, gate, a, heads, kv_heads, head_dim, v_dim, scale, window,
                            ctx.plan ? &w : nullptr, &ctx.ws);
    ctx.ops.linear(a, w_o, out, epi, epi == Ops::Add);
  }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override {
    if (!general) return MixerPart::forward_store(ctx, h, y);
    if (gated) return run_gated(ctx, h, y, Ops::Store);
    run_general(ctx, h, y, Ops::Store);
  }

  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    if (gated) return run_gated(ctx, h, x, Ops::Add);
    if (general) return run_general(ctx, h, x, Ops::Add);
    const int64_t M = h.t.shape[0];
    const int64_t width = nq + 2 * nk;
    Tensor q = ctx.buf("attn.q", ctx.act_dtype, {M, nq});
    const auto bound = ctx.binding(this);
    const Tensor pool = ctx.kv_pool(bound.first, bound.second);
    const Ops::CacheView view = ctx.cache_view(bound.first);
    Ops::Rotation rot;
    const bool has_rot = pos && pos->fused(rot);
    Tensor a = ctx.buf("attn.out", ctx.act_dtype, {M, nq});
    const bool fusable = !pos || has_rot;       // a position encoding without a fused form needs the 32-bit projections
    const float* qw = q_norm_w.ptr<float>();
    const float* kw = k_norm_w.ptr<float>();
    const AttentionWork w = work(ctx);
    const int n_kv_written = shares_kv ? 0 : kv_heads;
    if (fusable && !ctx.decode_only &&
        ctx.ops.qkv_prepared(h, w_qkv, qw, kw, eps, rot, ctx.positions, ctx.slots, view, pool, q, heads, n_kv_written, head_dim)) {
      // a step of many tokens: the projection's epilogue prepared q and wrote the cache
      ctx.ops.attention(w, ctx.ws, view, q, pool, a, heads, kv_heads, head_dim, scale, window);
      ctx.ops.linear(a, w_o, x, Ops::Add, true);
      return;
    }
    Tensor qkv = ctx.buf("attn.qkv", DType::F32, {M, width});
    ctx.ops.linear(h, w_qkv, qkv, Ops::Store);
    if (fusable && ctx.ops.attention_from_projections(w, ctx.ws, view, qkv, qw, kw, eps, rot, pool, !shares_kv, a, heads,
                                                      kv_heads, head_dim, scale, window)) {
      // a step of single tokens: one kernel did it all
      ctx.ops.linear(a, w_o, x, Ops::Add, true);
      return;
    }
    if (pos && !has_rot) {
      // a position encoding without a fused form works on the 32-bit projections, after the per-head
      // norm (as in the fused order: norm, then position)
      if (qw || kw) {
        ctx.ops.qk_norm_inplace(qkv, qw, kw, eps, heads, n_kv_written, head_dim);
        qw = kw = nullptr;
      }
      Tensor qv = qkv.cols(0, nq);
      qv.ndim = 3;
      qv.shape[0] = M; qv.shape[1] = heads; qv.shape[2] = head_dim;
      qv.stride[0] = width; qv.stride[1] = head_dim; qv.stride[2] = 1;
      Tensor kv;
      if (!shares_kv) {
        kv = qkv.cols(nq, nk);
        kv.ndim = 3;
        kv.shape[0] = M; kv.shape[1] = kv_heads; kv.shape[2] = head_dim;
        kv.stride[0] = width; kv.stride[1] = head_dim; kv.stride[2] = 1;
      }
      ctx.ops.flush();
      pos->apply(ctx, qv, kv);
    }
    ctx.ops.qk_norm_rope_kv_write(qkv, qw, kw, eps, rot, ctx.positions, ctx.slots, view, pool, q, heads, n_kv_written, head_dim);
    ctx.ops.attention(w, ctx.ws, view, q, pool, a, heads, kv_heads, head_dim, scale, window);
    ctx.ops.linear(a, w_o, x, Ops::Add, true);
  }

  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_qkv", w_qkv}, {"w_o", w_o}, {"q_norm_w", q_norm_w}, {"k_norm_w", k_norm_w}, {"b_qkv", b_qkv}};
  }
  int64_t hidden = 0, nq = 0, nk = 0, nv = 0, no = 0, ng = 0;
  int heads = 0, kv_heads = 0, head_dim = 0, v_dim = 0, window = 0, temp_every = 0;
  bool qk_norm = true, shares_kv = false, general = false, bias = false;
  bool gated = false;             // any of the four below: the gated kernels run
  bool has_sink = false;          // `sink`: exp(sink_h) joins the softmax's denominator (tensor `sink_tensor`, default prefix.sink)
  int gate_mode = 0;              // `gate` "entry" (1) / "head" (2): the heads' outputs times sigmoid(W_g h) (tensor `gate_tensor`, prefix.g)
  bool values_from_keys = false;  // `values_from_keys`: no value projection; a value is its key as projected
  int mix_mode = 0;               // `v_mix` "first" (1): the values are kept for later layers; "mix" (2): v <- (1 - l) v + l kept
  std::string n_qn, n_kn, n_sink, n_gate, n_vmix;
  bool vmix_named = false;
  Tensor sink, mix_lambda;
  Tensor b_qkv;      // `bias`: the biases of q, k and v side by side, 32-bit
  float eps = 1e-6f, scale = 1.f, softcap = 0.f, temp_coef = 0.f;
  std::string n_q, n_k, n_v, n_o;
  std::shared_ptr<PositionPart> pos;
  Tensor w_qkv, w_o, q_norm_w, k_norm_w;
};

// x += mixer(norm1(x)); x += ffn(norm2(x)).  The mixer and the feed-forward add into x
// themselves, so the residual sum happens in 32-bit in their last kernel.  That kernel may leave
// part of the sum to the norm that reads x next; before a part that does not read x through the
// kernels' own object, the sum is completed.
class PreNormBlock final : public BlockPart {
 public:
  PreNormBlock(const std::string& prefix, const PartChildren& c) : BlockPart(prefix) {
    for (const auto& kv : c) {
      if (kv.first == "norm1") norm1 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "mixer") mixer = std::dynamic_pointer_cast<MixerPart>(kv.second);
      if (kv.first == "norm2") norm2 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "ffn") ffn = std::dynamic_pointer_cast<FeedForwardPart>(kv.second);
    }
    if (!norm1 || !mixer) throw ConfigError("block 'pre_norm' needs norm1 and mixer parts (norm2 and ffn are optional)");
    if ((ffn != nullptr) != (norm2 != nullptr)) throw ConfigError("block 'pre_norm': norm2 and ffn come together or not at all");
  }
  const char* kind_name() const override { return "pre_norm"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    if (!ffn) return {norm1, mixer};
    return {norm1, mixer, norm2, ffn};
  }
  std::vector<std::string> child_slots() const override {
    if (!ffn) return {"norm1", "mixer"};
    return {"norm1", "mixer", "norm2", "ffn"};
  }
  void forward(StepContext& ctx, const Tensor& x) override {
    if (!norm1->reads_through_ops()) ctx.ops.flush();
    Rows h = norm1->forward(ctx, x, nullptr, 0, mixer->takes_lazy_norm() && norm1->can_be_lazy());
    if (!mixer->reads_through_ops()) ctx.ops.flush();
    mixer->forward(ctx, h, x);
    if (!ffn) return;      // a layer without a feed-forward
    if (!norm2->reads_through_ops()) ctx.ops.flush();
    h = norm2->forward(ctx, x, nullptr, 0, ffn->takes_lazy_norm() && norm2->can_be_lazy());
    if (!ffn->reads_through_ops()) ctx.ops.flush();
    ffn->forward(ctx, h, x);
  }
  std::shared_ptr<NormPart> norm1, norm2;
  std::shared_ptr<MixerPart> mixer;
  std::shared_ptr<FeedForwardPart> ffn;
};

// down(act(up h)) with act = xIELU and its two learned numbers (p, q) in the tensor `act`:
//   z > 0: softplus(p) z^2 + z / 2;   z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2.
// The first product leaves 32-bit sums, the activation is taken in 32-bit and rounded once to the compute dtype.
// Tensor names: prefix + ".up", ".down", ".act" unless the parameters `up`, `down`, `act` give them in full.
class DenseFFN final : public FeedForwardPart {
 public:
  DenseFFN(const std::string& prefix, const Json& p) : FeedForwardPart(prefix) {
    hidden = param_int(p, "hidden");
    intermediate = param_int(p, "intermediate");
    const std::string act = p.has("activation") ? p.at("activation").as_string() : "xielu";
    if (act != "xielu") throw ConfigError("dense feed-forward: activation '" + act + "' is not served (only 'xielu')");
    if (hidden <= 0 || intermediate <= 0) throw ConfigError("dense feed-forward: sizes must be positive");
    n_up = tensor_name(p, "up", prefix, "up");
    n_down = tensor_name(p, "down", prefix, "down");
    n_act = tensor_name(p, "act", prefix, "act");
  }
  const char* kind_name() const override { return "dense"; }
  bool takes_lazy_norm() const override { return true; }       // h goes into the up product and nowhere else
  bool reads_through_ops() const override { return true; }
  bool can_store() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed up, down, act;
    up.shape = {intermediate, hidden};
    down.shape = {hidden, intermediate};
    act.shape = {2};
    act.role = TensorNeed::Vector;
    act.a = 0.5;
    act.b = 0.2;
    return {{n_up, up}, {n_down, down}, {n_act, act}};
  }
  void load(WeightSource& src) override {
    const auto t = tensors();
    w_up = src.fetch(n_up, t[0].second);
    w_down = src.fetch(n_down, t[1].second);
    act = src.fetch(n_act, t[2].second);
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor z = ctx.buf("ffn.z", DType::F32, {M, intermediate});
    ctx.ops.linear(h, w_up, z, Ops::Store);
    Tensor y = ctx.buf("ffn.y", ctx.act_dtype, {M, intermediate});
    ctx.ops.xielu(z, act, y);
    ctx.ops.linear(y, w_down, out, epi, epi == Ops::Add);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x, Ops::Add); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override { run(ctx, h, y, Ops::Store); }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w_up", w_up}, {"w_down", w_down}, {"act", act}}; }
  int64_t hidden = 0, intermediate = 0;
  std::string n_up, n_down, n_act;
  Tensor w_up, w_down, act;
};

// The mLSTM cell.  With q = W_q h / sqrt(dk), k = W_k h (heads x dk), v = W_v h (heads x dv) and per head a log
// input gate i = cap tanh((W_i h + b_i) / cap) and a log forget gate f = logsigmoid(cap tanh((W_f h + b_f) / cap)):
//   m_t = max(f + m_(t-1), i);  S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T;  n_t likewise with k;
//   o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6),
// S, n and m starting at zero.  Each head's o is divided by its root mean square, the heads are multiplied by the
// vector `norm` and by sigmoid(W_g h), and W_o maps them back.  q, k, v, the output gate and the two gates'
// pre-activations come from one product with the stacked weight [q; k; v; g; i; f].  The memory (S, n, m per head)
// is per-request state in 32-bit: a request's slot, zeroed when it is admitted; each run of the layer has its own.
// Tensor names: prefix + ".q", ".k", ".v", ".g", ".o", ".norm", ".i", ".i.b", ".f", ".f.b".
class MLSTM final : public MixerPart {
 public:
  MLSTM(const std::string& prefix, const Json& p) : MixerPart(prefix) {
    hidden = param_int(p, "hidden");
    heads = (int)param_int(p, "heads");
    dk = (int)param_int(p, "head_dim");
    dv = p.has("v_head_dim") ? (int)param_int(p, "v_head_dim") : dk;
    cap = (float)param_float(p, "gate_cap");
    eps = (float)param_float(p, "eps");
    if (heads <= 0 || dk <= 0 || dv <= 0 || hidden <= 0) throw ConfigError("mlstm: sizes must be positive");
    if (dk > 256) throw ConfigError("mlstm: a key size of " + std::to_string(dk) + " is not served (up to 256)");
    const int padded = dk <= 32 ? 32 : dk <= 64 ? 64 : dk <= 128 ? 128 : 256;      // the rows the scan kernel holds
    if (2 * padded + dv > 1016)
      throw ConfigError("mlstm: a value size of " + std::to_string(dv) + " beside a key size of " + std::to_string(dk) +
                        " is not served (the scan stages sixteen tokens' q, k and v in 64 KB)");
    if (!(cap > 0.f)) throw ConfigError("mlstm: gate_cap must be positive");
    nq = (int64_t)heads * dk;
    nv = (int64_t)heads * dv;
    width = 2 * nq + 2 * nv + 2 * heads;
  }
  const char* kind_name() const override { return "mlstm"; }
  bool takes_lazy_norm() const override { return true; }       // h goes into the stacked projection and nowhere else
  bool reads_through_ops() const override { return true; }
  bool can_store() const override { return true; }
  std::string name(const char* t) const { return join(prefix, t); }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed qk, v, o, gate, bias, nw;
    qk.shape = {nq, hidden};
    v.shape = {nv, hidden};
    o.shape = {hidden, nv};
    gate.shape = {heads, hidden};
    bias.shape = {heads};
    bias.role = TensorNeed::Vector;
    bias.b = 1.0;
    nw.shape = {nv};
    nw.role = TensorNeed::Vector;
    nw.a = 1.0;
    nw.b = 0.1;
    return {{name("q"), qk}, {name("k"), qk}, {name("v"), v}, {name("g"), v}, {name("o"), o}, {name("norm"), nw},
            {name("i"), gate}, {name("i.b"), bias}, {name("f"), gate}, {name("f.b"), bias}};
  }
  void load(WeightSource& src) override {
    w_in = src.alloc(src.matrix_dtype, {width, hidden});
    src.fill(name("q"), w_in.rows(0, nq));
    src.fill(name("k"), w_in.rows(nq, nq));
    src.fill(name("v"), w_in.rows(2 * nq, nv));
    src.fill(name("g"), w_in.rows(2 * nq + nv, nv));
    src.fill(name("i"), w_in.rows(2 * nq + 2 * nv, heads));
    src.fill(name("f"), w_in.rows(2 * nq + 2 * nv + heads, heads));
    TensorNeed o, bias, nw;
    o.shape = {hidden, nv};
    bias.shape = {heads};
    bias.role = TensorNeed::Vector;
    nw.shape = {nv};
    nw.role = TensorNeed::Vector;
    w_o = src.fetch(name("o"), o);
    norm_w = src.fetch(name("norm"), nw);
    b_i = src.fetch(name("i.b"), bias);
    b_f = src.fetch(name("f.b"), bias);
  }
  bool has_cache() const override { return true; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {heads, (int64_t)dk * dv + dk + 1};
    return n;
  }
  // A step with a long portion: every entry's tokens in chunks of CHUNK (the cell's recurrence runs inside the chunks
  // side by side and from chunk to chunk element-wise), from CHUNK_FROM tokens on, where three chunks or more make up
  // for walking the tokens twice.  The lists are the same for every mLSTM of the model; the first one builds them.
  static constexpr int CHUNK = 64, CHUNK_FROM = 192;
  void plan(StepPlan& plan) const override {
    if (plan.decode_only() || plan.has("mlstm.chunks")) return;
    const auto& entries = plan.entries();
    int longest = 0;
    size_t n_chunks = 0;
    for (const auto& e : entries) {
      longest = std::max(longest, e.n_tokens);
      n_chunks += (size_t)(e.n_tokens + CHUNK - 1) / CHUNK;
    }
    if (longest < CHUNK_FROM) return;
    int* chunks = plan.ints("mlstm.chunks", 4 * n_chunks);
    int* spans = plan.ints("mlstm.spans", 2 * entries.size());
    int c = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
      const auto& e = entries[i];
      const int n = (e.n_tokens + CHUNK - 1) / CHUNK;
      spans[2 * i] = c;
      spans[2 * i + 1] = n;
      for (int k = 0; k < n; ++k, ++c) {
        chunks[4 * c] = (int)i;
        chunks[4 * c + 1] = e.row0 + k * CHUNK;
        chunks[4 * c + 2] = std::min(CHUNK, e.n_tokens - k * CHUNK);
        chunks[4 * c + 3] = (k == 0 ? 1 : 0) | (k == n - 1 ? 2 : 0);
      }
    }
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor proj = ctx.buf("mlstm.proj", DType::F32, {M, width});
    ctx.ops.linear(h, w_in, proj, Ops::Store);
    const auto bound = ctx.binding(this);
    const Tensor state = ctx.state(bound.first, bound.second);
    Tensor o = ctx.buf("mlstm.o", DType::F32, {M, nv});
    Ops::MlstmColumns cols;
    cols.q = 0;
    cols.k = (int)nq;
    cols.v = (int)(2 * nq);
    cols.i = (int)(2 * nq + 2 * nv);
    cols.f = cols.i + heads;
    ctx.ops.mlstm_scan(proj, cols, b_i, b_f, state, ctx.entry_meta, (int)ctx.entries.size(), o, heads, dk, dv, cap,
                       (float)(1.0 / std::sqrt((double)dk)), ctx.planned("mlstm.chunks"), (int)(ctx.planned_size("mlstm.chunks") / 4),
                       ctx.planned("mlstm.spans"), &ctx.ws);
    Tensor a = ctx.buf("mlstm.gated", ctx.act_dtype, {M, nv});
    ctx.ops.gated_head_norm(o, proj, (int)(2 * nq + nv), norm_w, eps, a, heads, dv);
    ctx.ops.linear(a, w_o, out, epi, epi == Ops::Add);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x, Ops::Add); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override { run(ctx, h, y, Ops::Store); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_in", w_in}, {"w_o", w_o}, {"norm_w", norm_w}, {"b_i", b_i}, {"b_f", b_f}};
  }
  int64_t hidden = 0, nq = 0, nv = 0, width = 0;
  int heads = 0, dk = 0, dv = 0;
  float cap = 1.f, eps = 1e-6f;
  Tensor w_in, w_o, norm_w, b_i, b_f;
};

// A parallel layer: h = norm1(x); x += s1 * mixer(h) + s2 * ffn(h).  One norm feeds both branches; each branch's
// output is scaled per channel by a learned vector (`scale1`, `scale2`: the tensors' names after the prefix, absent:
// no scaling) before the two are added to the residual together, in 32-bit.  Without a feed-forward the mixer alone
// is added.  Branches that can write their output apart from the residual do so; others add into a zeroed buffer.
class ParallelBlock final : public BlockPart {
 public:
  ParallelBlock(const std::string& prefix, const Json& p, const PartChildren& c) : BlockPart(prefix) {
    for (const auto& kv : c) {
      if (kv.first == "norm1") norm1 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "mixer") mixer = std::dynamic_pointer_cast<MixerPart>(kv.second);
      if (kv.first == "ffn") ffn = std::dynamic_pointer_cast<FeedForwardPart>(kv.second);
    }
    if (!norm1 || !mixer) throw ConfigError("block 'parallel' needs norm1 and mixer parts (ffn is optional)");
    dim = param_int(p, "dim");
    if (p.has("scale1")) scale1 = join(prefix, p.at("scale1").as_string());
    if (p.has("scale2")) scale2 = join(prefix, p.at("scale2").as_string());
  }
  const char* kind_name() const override { return "parallel"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    std::vector<std::shared_ptr<Part>> v = {norm1, mixer};
    if (ffn) v.push_back(ffn);
    return v;
  }
  std::vector<std::string> child_slots() const override {
    std::vector<std::string> v = {"norm1", "mixer"};
    if (ffn) v.push_back("ffn");
    return v;
  }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    TensorNeed n;
    n.shape = {dim};
    n.role = TensorNeed::Vector;
    n.a = 1.0;
    n.b = 0.3;
    if (!scale1.empty()) t.emplace_back(scale1, n);
    if (!scale2.empty()) {
      n.optional = !ffn;     // a layer without a feed-forward has nothing for it to scale
      t.emplace_back(scale2, n);
    }
    return t;
  }
  void load(WeightSource& src) override {
    TensorNeed n;
    n.shape = {dim};
    n.role = TensorNeed::Vector;
    if (!scale1.empty()) s1 = src.fetch(scale1, n);
    if (!scale2.empty() && ffn) s2 = src.fetch(scale2, n);
  }
  void forward(StepContext& ctx, const Tensor& x) override {
    if (!norm1->reads_through_ops()) ctx.ops.flush();
    // each branch feeds h to one product: where a product can take the norm in (a step of few rows), the rows stay
    // uncomputed and each branch's first product norms them itself; the first product that cannot computes them for all
    bool lazy = norm1->can_be_lazy() && mixer->takes_lazy_norm() && (!ffn || ffn->takes_lazy_norm());
    const Rows h = norm1->forward(ctx, x, nullptr, 0, lazy);
    const int64_t M = x.shape[0];
    Tensor y1 = ctx.buf("parallel.y1", DType::F32, {M, dim});
    if (!mixer->reads_through_ops()) ctx.ops.flush();
    if (mixer->can_store()) {
      mixer->forward_store(ctx, h, y1);
    } else {
      ctx.ops.fill_zero(y1.data, y1.bytes());
      mixer->forward(ctx, h, y1);
    }
    Tensor y2;
    if (ffn) {
      y2 = ctx.buf("parallel.y2", DType::F32, {M, dim});
      if (!ffn->reads_through_ops()) ctx.ops.flush();
      if (ffn->can_store()) {
        ffn->forward_store(ctx, h, y2);
      } else {
        ctx.ops.fill_zero(y2.data, y2.bytes());
        ffn->forward(ctx, h, y2);
      }
    }
    ctx.ops.scaled_add(x, y1, s1, y2, s2);
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"s1", s1}, {"s2", s2}}; }
  std::shared_ptr<NormPart> norm1;
  std::shared_ptr<MixerPart> mixer;
  std::shared_ptr<FeedForwardPart> ffn;
  int64_t dim = 0;
  std::string scale1, scale2;
  Tensor s1, s2;
};

// x += table[row]: a learned vector onto every token of the step (what a looped run of layers adds before each
// of its passes: the pass number is the row).  `tensor`: the table's name, [rows, dim]; several such blocks share it.
class AddVectorBlock final : public BlockPart {
 public:
  AddVectorBlock(const std::string& prefix, const Json& p) : BlockPart(prefix) {
    dim = param_int(p, "dim");
    rows = param_int(p, "rows");
    row = param_int(p, "row");
    name = tensor_name(p, "tensor", prefix, "weight");
    if (row < 0 || row >= rows) throw ConfigError("block 'add_vector': row " + std::to_string(row) + " is outside its " + std::to_string(rows) + " rows");
  }
  const char* kind_name() const override { return "add_vector"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    n.shape = {rows, dim};
    n.role = TensorNeed::Vector;
    n.b = 0.5;
    return {{name, n}};
  }
  void load(WeightSource& src) override { table = src.fetch(name, tensors()[0].second); }
  void forward(StepContext& ctx, const Tensor& x) override { ctx.ops.add_row(x, table.rows(row, 1)); }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"table", table}}; }
  int64_t dim = 0, rows = 0, row = 0;
  std::string name;
  Tensor table;
};

// Rotation of the first `dims` entries of a head in the half-split layout (entry i turns with entry i + dims / 2 by
// the angle pos * f_i, f_i = base^(-2i / dims)); the rest of the head passes.  `scaling` {factor, original, fast, slow}
// interpolates the frequencies as YaRN does: with dim(t) = dims ln(original / (2 pi t)) / (2 ln base),
// lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
// the frequency is f_i / factor * ramp_i + f_i (1 - ramp_i), and cosine and sine are multiplied by 0.1 ln(factor) + 1.
// Frequencies and, for the positions an engine serves, cosines and sines are built on the host in double precision
// and rounded once; a table is immutable and lives as long as the part (captured graphs hold its address).
class RotaryPartial final : public PositionPart {
 public:
  RotaryPartial(const std::string& prefix, const Json& p) : PositionPart(prefix) {
    dims = (int)param_int(p, "dims");
    base = param_float(p, "base");
    if (dims < 0 || dims % 2) throw ConfigError("rotary: " + std::to_string(dims) + " rotated entries: must be even and not negative");
    if (!(base > 0.0)) throw ConfigError("rotary: base must be positive");
    if (p.has("scaling")) {
      const Json& sc = p.at("scaling");
      factor = param_float(sc, "factor");
      original = param_float(sc, "original");
      fast = param_float(sc, "fast");
      slow = param_float(sc, "slow");
      if (!(factor > 0.0) || !(original > 0.0) || !(fast > 0.0) || !(slow > 0.0))
        throw ConfigError("rotary: scaling factor, original, fast and slow must be positive");
      scaled = true;
    }
    const int half = dims / 2;
    freq.resize(half);
    for (int i = 0; i < half; ++i) freq[i] = std::pow(base, -2.0 * i / dims);
    if (scaled) {
      const double pi = 3.14159265358979323846;
      auto dim_of = [&](double turns) { return dims * std::log(original / (2.0 * pi * turns)) / (2.0 * std::log(base)); };
      const double lo = std::max(std::floor(dim_of(fast)), 0.0);
      const double hi = std::min(std::ceil(dim_of(slow)), (double)(dims - 1));
      for (int i = 0; i < half; ++i) {
        const double ramp = std::min(1.0, std::max(0.0, (i - lo) / std::max(hi - lo, 0.001)));
        freq[i] = freq[i] / factor * ramp + freq[i] * (1.0 - ramp);
      }
      mag = 0.1 * std::log(factor) + 1.0;
    }
  }
  const char* kind_name() const override { return "rope_partial"; }
  void prepare(Ops&, int max_seq) override {
    std::lock_guard<std::mutex> lock(g_rope_mutex);
    const int half = dims / 2;
    if (half == 0) return;
    if (!inv_freq.data()) {
      std::vector<float> f32(freq.begin(), freq.end());
      inv_freq = DeviceBuffer((size_t)half * 4);
      RotaryNeox::upload(inv_freq.data(), f32.data(), (size_t)half * 4);
    }
    if (max_seq <= table_len) return;
    std::vector<float> host((size_t)max_seq * half * 2);
    for (int p = 0; p < max_seq; ++p)
      for (int i = 0; i < half; ++i) {
        const double a = (double)p * freq[i];
        host[((size_t)p * half + i) * 2] = (float)(std::cos(a) * mag);
        host[((size_t)p * half + i) * 2 + 1] = (float)(std::sin(a) * mag);
      }
    tables.emplace_back(host.size() * 4);
    RotaryNeox::upload(tables.back().data(), host.data(), host.size() * 4);
    table_len = max_seq;
  }
  bool fused(Ops::Rotation& rot) const override {
    std::lock_guard<std::mutex> lock(g_rope_mutex);
    if (dims == 0 || !inv_freq.data()) return false;
    rot.inv_freq = (const float*)inv_freq.data();
    rot.table = tables.empty() ? nullptr : (const float*)tables.back().data();
    rot.table_len = table_len;
    rot.dims = dims;
    rot.mag = (float)mag;
    return true;
  }
  void apply(StepContext&, const Tensor&, const Tensor&) override {
    throw EngineError("the partial rotation is applied by the kernels that prepare queries and keys (fused)");
  }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    if (!inv_freq.data()) return {};
    std::vector<std::pair<std::string, Tensor>> h = {{"inv_freq", Tensor(inv_freq.data(), DType::F32, {dims / 2})}};
    if (table_len) h.emplace_back("table", Tensor(tables.back().data(), DType::F32, {table_len, dims / 2, 2}));
    return h;
  }
  int dims = 0;
  double base = 10000.0, factor = 1.0, original = 0.0, fast = 0.0, slow = 0.0, mag = 1.0;
  bool scaled = false;
  std::vector<double> freq;
  DeviceBuffer inv_freq;
  std::vector<DeviceBuffer> tables;     // oldest first; the last one is read
  int table_len = 0;
};

// A causal convolution over time on every channel of the rows it is given: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros
// before a sequence's start, no bias.  `segments`: [[tensor name, channels], ...], the taps [channels, taps] of runs of
// channels side by side (the parts of a fused projection each bring their own tensor).  The last taps - 1 rows of every
// request are its state (32-bit, zeroed at admission: the zeros before the start).
class ShortConv final : public FilterPart {
 public:
  ShortConv(const std::string& prefix, const Json& p) : FilterPart(prefix) {
    taps = (int)param_int(p, "taps");
    if (taps < 1) throw ConfigError("short_conv: taps must be at least 1");
    const Json* seg = p.find("segments");
    if (!seg || seg->type() != Json::Array || seg->size() == 0) throw ConfigError("short_conv: 'segments' must list [tensor, channels] pairs");
    for (const Json& s : seg->items()) {
      if (s.type() != Json::Array || s.size() != 2 || s[0].type() != Json::String || !s[1].is_number() || s[1].as_int() <= 0)
        throw ConfigError("short_conv: a segment is [tensor name, channels]");
      segments.emplace_back(s[0].as_string(), s[1].as_int());
      channels += s[1].as_int();
    }
  }
  const char* kind_name() const override { return "short_conv"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    for (const auto& s : segments) {
      TensorNeed n;
      n.shape = {s.second, (int64_t)taps};
      n.role = TensorNeed::Vector;
      n.a = 1.0 / taps;
      n.b = 0.3;
      t.emplace_back(s.first, n);
    }
    return t;
  }
  void load(WeightSource& src) override {
    w = src.alloc(DType::F32, {channels, (int64_t)taps});
    int64_t at = 0;
    for (const auto& s : segments) {
      src.fill(s.first, w.rows(at, s.second));
      at += s.second;
    }
  }
  bool has_cache() const override { return taps > 1; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {(int64_t)taps - 1, channels};
    return n;
  }
  Tensor state_of(StepContext& ctx) const {
    if (taps == 1) return Tensor();
    const auto bound = ctx.binding(this);
    return ctx.state(bound.first, bound.second);
  }
  void forward(StepContext& ctx, const Tensor& u, const Tensor& out) override {
    ctx.ops.short_conv(u, w, state_of(ctx), ctx.entry_meta, (int)ctx.entries.size(), ctx.slots, ctx.positions, out);
  }
  bool fused(StepContext& ctx, Ops::ShortConv& conv) override {
    conv.taps = w;
    conv.state = state_of(ctx);
    conv.entry_meta = ctx.entry_meta;
    conv.n_entries = (int)ctx.entries.size();
    conv.entry_of = ctx.slots;
    return true;
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w", w}}; }
  int taps = 1;
  int64_t channels = 0;
  std::vector<std::pair<std::string, int64_t>> segments;
  Tensor w;
};

// Differential attention.  Every one of the `heads` query heads holds two maps: q has heads x 2 x head_dim rows, k has
// kv_heads x 2 x head_dim (head by head as [map 1, map 2]), v has kv_heads x v_head_dim; query head h reads key/value
// head floor(h / (heads / kv_heads)).  Behind the fused projection: the child `conv` (a filter over time, optional) on all
// its channels, then per head and map an RMS norm over head_dim (weights `q_norm`, `k_norm` of size head_dim, shared by
// all heads and maps; `qk_norm` false: none) and the rotation of the child `pos` (optional); v is left alone.  Each map is
// a softmax attention of its own, scores (q . k) * scale over the keys that are not later and lie in the query's block of
// `block` positions counted from 0 (0: no blocks; `window` likewise optional); both read the same values.  With a1, a2 the
// maps' outputs and lambda = exp(sum(lq1 * lk1)) - exp(sum(lq2 * lk2)) + diff (vectors of size head_dim, one number a
// layer, formed once when the weights load): o = a1 - lambda a2, divided by its root mean square over v_head_dim (eps, no
// weight), times 1 - diff; then the output projection.  Scores, softmax, lambda and the norms are 32-bit.
class DiffAttention final : public MixerPart {
 public:
  DiffAttention(const std::string& prefix, const Json& p, const PartChildren& children) : MixerPart(prefix) {
    hidden = param_int(p, "hidden");
    heads = (int)param_int(p, "heads");
    kv_heads = p.has("kv_heads") ? (int)param_int(p, "kv_heads") : heads;
    dk = (int)param_int(p, "head_dim");
    dv = p.has("v_head_dim") ? (int)param_int(p, "v_head_dim") : dk;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads)
      throw ConfigError("diff_attention: heads " + std::to_string(heads) + " not a multiple of kv_heads " + std::to_string(kv_heads));
    if (dk < 1 || dk > 256 || dv < 1 || dv > 256)
      throw ConfigError("diff_attention: key size " + std::to_string(dk) + " / value size " + std::to_string(dv) + " are not served (up to 256)");
    diff = param_float(p, "diff");
    eps = (float)(p.has("eps") ? param_float(p, "eps") : 1e-6);
    scale = p.has("scale") ? (float)param_float(p, "scale") : (float)(1.0 / std::sqrt((double)dk));
    block = p.has("block") ? (int)param_int(p, "block") : 0;
    window = p.has("window") ? (int)param_int(p, "window") : 0;
    if (block < 0 || window < 0) throw ConfigError("diff_attention: block and window must not be negative");
    qk_norm = p.has("qk_norm") ? p.at("qk_norm").as_bool() : true;
    for (const auto& c : children) {
      if (c.first == "pos") pos = std::dynamic_pointer_cast<PositionPart>(c.second);
      if (c.first == "conv") conv = std::dynamic_pointer_cast<FilterPart>(c.second);
    }
    if (!pos && p.has("pos")) pos = std::dynamic_pointer_cast<PositionPart>(build_part("pos", PartSpec::from_json(p.at("pos")), prefix));
    if (!conv && p.has("conv")) conv = std::dynamic_pointer_cast<FilterPart>(build_part("filter", PartSpec::from_json(p.at("conv")), prefix));
    nq = (int64_t)heads * 2 * dk;
    nk = (int64_t)kv_heads * 2 * dk;
    nv = (int64_t)kv_heads * dv;
    no = (int64_t)heads * dv;
    n_q = tensor_name(p, "q", prefix, "q");
    n_k = tensor_name(p, "k", prefix, "k");
    n_v = tensor_name(p, "v", prefix, "v");
    n_o = tensor_name(p, "o", prefix, "o");
    n_qn = tensor_name(p, "q_norm", prefix, "q.norm");
    n_kn = tensor_name(p, "k_norm", prefix, "k.norm");
    for (int i = 0; i < 4; ++i) {
      static const char* keys[4] = {"lq1", "lk1", "lq2", "lk2"};
      n_l[i] = tensor_name(p, keys[i], prefix, keys[i]);
    }
  }
  const char* kind_name() const override { return "diff_attention"; }
  bool can_store() const override { return true; }
  bool takes_lazy_norm() const override { return true; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    std::vector<std::shared_ptr<Part>> v;
    if (pos) v.push_back(pos);
    if (conv) v.push_back(conv);
    return v;
  }
  std::vector<std::string> child_slots() const override {
    std::vector<std::string> v;
    if (pos) v.push_back("pos");
    if (conv) v.push_back("conv");
    return v;
  }
  TensorNeed vector_need(double a, double b) const {
    TensorNeed n;
    n.shape = {dk};
    n.role = TensorNeed::Vector;
    n.a = a;
    n.b = b;
    return n;
  }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    TensorNeed q, k, v, o;
    q.shape = {nq, hidden};
    k.shape = {nk, hidden};
    v.shape = {nv, hidden};
    o.shape = {hidden, no};
    t.emplace_back(n_q, q);
    t.emplace_back(n_k, k);
    t.emplace_back(n_v, v);
    t.emplace_back(n_o, o);
    if (qk_norm) {
      t.emplace_back(n_qn, vector_need(1.0, 0.1));
      t.emplace_back(n_kn, vector_need(1.0, 0.1));
    }
    for (int i = 0; i < 4; ++i) t.emplace_back(n_l[i], vector_need(0.0, 0.1));
    return t;
  }
  void load(WeightSource& src) override {
    w_qkv = src.alloc(src.matrix_dtype, {nq + nk + nv, hidden});
    src.fill(n_q, w_qkv.rows(0, nq));
    src.fill(n_k, w_qkv.rows(nq, nk));
    src.fill(n_v, w_qkv.rows(nq + nk, nv));
    TensorNeed o;
    o.shape = {hidden, no};
    w_o = src.fetch(n_o, o);
    if (qk_norm) {
      q_norm_w = src.fetch(n_qn, vector_need(1.0, 0.1));
      k_norm_w = src.fetch(n_kn, vector_need(1.0, 0.1));
    }
    Tensor l[4];
    for (int i = 0; i < 4; ++i) l[i] = src.fetch(n_l[i], vector_need(0.0, 0.1));
    lambda = lambda_of(l, dk, diff, src.to_host);
  }
  // exp(sum(lq1 * lk1)) - exp(sum(lq2 * lk2)) + diff, sums and exponentials in 32-bit
  static float lambda_of(const Tensor l[4], int dk, double diff, bool on_host);
  bool has_cache() const override { return true; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::PagedKV;
    n.kv_heads = kv_heads;
    n.head_dim = 2 * dk;          // a row's two maps side by side
    n.v_dim = dv != 2 * dk ? dv : 0;
    n.window = window;
    n.block = block;
    return n;
  }
  // The lists of the matrix-core kernels: tiles of TILE_ROWS query rows over the entries of several tokens, and the rows
  // of single-token entries.  Every such mixer of a model asks for the same lists; the first one builds them.
  static constexpr int TILE_ROWS = 64;
  void plan(StepPlan& plan) const override {
    if (plan.decode_only() || plan.has("dattn.tiles")) return;
    const auto& entries = plan.entries();
    size_t n_tiles = 0, n_rows = 0;
    for (const auto& e : entries) {
      if (e.n_tokens > 1) n_tiles += (size_t)(e.n_tokens + TILE_ROWS - 1) / TILE_ROWS;
      else ++n_rows;
    }
    int* tiles = plan.ints("dattn.tiles", 3 * n_tiles);
    int* rows = plan.ints("dattn.rows", n_rows);
    struct Tile { int keys, entry, row, n; };
    std::vector<Tile> order;
    order.reserve(n_tiles);
    size_t r = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
      const auto& e = entries[i];
      if (e.n_tokens == 1) {
        rows[r++] = e.row0;
        continue;
      }
      for (int q0 = 0; q0 < e.n_tokens; q0 += TILE_ROWS) {
        const int n = std::min(TILE_ROWS, e.n_tokens - q0);
        const int last = e.start + q0 + n - 1;                       // the tile's last position, and how many keys it sees
        order.push_back({block > 0 ? last % block + 1 : last + 1, (int)i, e.row0 + q0, n});
      }
    }
    // from the tile that walks the most keys to the one that walks the fewest: the long ones start first
    std::stable_sort(order.begin(), order.end(), [](const Tile& a, const Tile& b) { return a.keys > b.keys; });
    for (size_t t = 0; t < order.size(); ++t) {
      tiles[3 * t] = order[t].entry;
      tiles[3 * t + 1] = order[t].row;
      tiles[3 * t + 2] = order[t].n;
    }
  }
  Ops::DiffAttentionLists lists(const StepContext& ctx) const {
    Ops::DiffAttentionLists l;
    l.entry_meta = ctx.entry_meta;
    // a captured graph serves every later step of its shape: what it launches is sized for the longest sequence
    l.context = ctx.plan && ctx.plan->sized_for_longest() ? ctx.plan->max_seq() : ctx.max_context;
    l.ws = &ctx.ws;
    if (ctx.decode_only) {
      l.n_rows = (int)ctx.M;
      return l;
    }
    l.tiles = ctx.planned("dattn.tiles");
    l.n_tiles = (int)(ctx.planned_size("dattn.tiles") / 3);
    l.rows = ctx.planned("dattn.rows");
    l.n_rows = (int)ctx.planned_size("dattn.rows");
    return l;
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    const int64_t width = nq + nk + nv;
    Tensor qkv = ctx.buf("dattn.qkv", DType::F32, {M, width});
    ctx.ops.linear(h, w_qkv, qkv, Ops::Store);
    // the convolution inside the kernel that prepares queries and keys, where the filter has a form for that
    Ops::ShortConv taken;
    const bool conv_inside = conv && conv->fused(ctx, taken);
    if (conv && !conv_inside) {
      Tensor mixed = ctx.buf("dattn.conv", DType::F32, {M, width});
      conv->forward(ctx, qkv, mixed);
      qkv = mixed;
    }
    const auto bound = ctx.binding(this);
    const Tensor pool = ctx.kv_pool(bound.first, bound.second);
    const Ops::CacheView view = ctx.cache_view(bound.first);
    Ops::Rotation rot;
    if (pos && !pos->fused(rot)) throw EngineError("diff_attention: the position encoding '" + std::string(pos->kind_name()) + "' has no fused form");
    Tensor q = ctx.buf("dattn.q", ctx.act_dtype, {M, nq});
    ctx.ops.diff_qk_prep(qkv, q_norm_w.ptr<float>(), k_norm_w.ptr<float>(), eps, rot, ctx.positions, ctx.slots, view, pool, q, heads,
                         kv_heads, dk, dv, conv_inside ? &taken : nullptr);
    Tensor a = ctx.buf("dattn.out", ctx.act_dtype, {M, no});
    const Ops::DiffAttentionLists l = lists(ctx);
    ctx.ops.diff_attention(q, pool, view, ctx.positions, ctx.slots, a, heads, kv_heads, dk, dv, scale, block, window, lambda, eps,
                           (float)(1.0 - diff), ctx.plan ? &l : nullptr);
    ctx.ops.linear(a, w_o, out, epi, false);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x, Ops::Add); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override { run(ctx, h, y, Ops::Store); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_qkv", w_qkv}, {"w_o", w_o}, {"q_norm_w", q_norm_w}, {"k_norm_w", k_norm_w}};
  }
  int64_t hidden = 0, nq = 0, nk = 0, nv = 0, no = 0;
  int heads = 0, kv_heads = 0, dk = 0, dv = 0, block = 0, window = 0;
  bool qk_norm = true;
  double diff = 0.0;
  float eps = 1e-6f, scale = 1.f, lambda = 0.f;
  std::string n_q, n_k, n_v, n_o, n_qn, n_kn, n_l[4];
  std::shared_ptr<PositionPart> pos;
  std::shared_ptr<FilterPart> conv;
  Tensor w_qkv, w_o, q_norm_w, k_norm_w;
};

// A mixture of experts: `experts` small feed-forward layers W_down act(W_up h) without biases (tensors prefix + ".e<i>.up"
// [intermediate, hidden], ".e<i>.down"), of which each token uses the `top` with the largest scores.  Router logits
// W_router h and the scores (`score`: "sigmoid", or "softmax" over all experts) are 32-bit; `renormalize`: the chosen
// scores are divided by their sum.  `scale_input` true: the score multiplies the expert's input, the output is
// sum_e expert_e(s_e h); false: its output.  `activation`: "relu2", the square of relu.
class MoE final : public FeedForwardPart {
 public:
  MoE(const std::string& prefix, const Json& p, const PartChildren& children = {}) : FeedForwardPart(prefix) {
    hidden = param_int(p, "hidden");
    intermediate = param_int(p, "intermediate");
    experts = (int)param_int(p, "experts");
    top = (int)param_int(p, "top");
    if (hidden <= 0 || intermediate <= 0) throw ConfigError("moe: sizes must be positive");
    if (experts < 1 || experts > 1024) throw ConfigError("moe: " + std::to_string(experts) + " experts are not served (1 to 1024)");
    if (top < 1 || top > experts || top > 64)
      throw ConfigError("moe: top " + std::to_string(top) + " must lie between 1 and the number of experts (and at most 64)");
    if (hidden * 4 > 64 * 1024 || intermediate * 4 > 64 * 1024)
      throw ConfigError("moe: a width of " + std::to_string(hidden) + " / an expert size of " + std::to_string(intermediate) +
                        " is not served (a row of either must fit 64 KB)");
    const std::string act = p.has("activation") ? p.at("activation").as_string() : "relu2";
    if (act != "relu2" && act != "glu_clamped" && act != "glu_silu")
      throw ConfigError("moe: activation '" + act + "' is not served (relu2, glu_clamped, glu_silu)");
    gated = act != "relu2";
    act_kind = act == "glu_clamped" ? Ops::ClampedGlu : Ops::Silu;
    if (act == "glu_clamped") {
      limit = (float)param_float(p, "limit");
      alpha = p.has("alpha") ? (float)param_float(p, "alpha") : 1.702f;
      if (!(limit > 0.f)) throw ConfigError("moe: the activation's limit must be positive");
    }
    const std::string sc = p.has("score") ? p.at("score").as_string() : "sigmoid";
    if (sc != "sigmoid" && sc != "softmax" && sc != "softmax_chosen")
      throw ConfigError("moe: score '" + sc + "' is not served (sigmoid, softmax, softmax_chosen)");
    score = sc == "softmax" ? Ops::Softmax : sc == "softmax_chosen" ? Ops::SoftmaxChosen : Ops::Sigmoid;
    renormalize = p.has("renormalize") && p.at("renormalize").as_bool();
    scale_input = gated ? false : (!p.has("scale_input") || p.at("scale_input").as_bool());
    if (gated && p.has("scale_input") && p.at("scale_input").as_bool()) throw ConfigError("moe: gated experts take their weight on the output");
    n_router = tensor_name(p, "router", prefix, "router");
    // a grouped router: a correction on the scores for the choice only, groups of neighbouring experts of which the best are
    // kept, a factor on the weights, a floor under the sum they are divided by
    corrected = p.has("correction") && p.at("correction").as_bool();
    n_correction = tensor_name(p, "correction_tensor", prefix, "correction");
    if (p.has("groups")) {
      groups = (int)param_int(p.at("groups"), "count");
      keep = (int)param_int(p.at("groups"), "keep");
      if (groups < 1 || experts % groups || keep < 1 || keep > groups || (int64_t)keep * (experts / groups) < top)
        throw ConfigError("moe: " + std::to_string(groups) + " groups of which " + std::to_string(keep) + " are kept do not fit " +
                          std::to_string(experts) + " experts and top " + std::to_string(top));
    }
    weight_scale = p.has("weight_scale") ? (float)param_float(p, "weight_scale") : 1.f;
    sum_floor = p.has("sum_floor") ? (float)param_float(p, "sum_floor") : 0.f;
    if ((corrected || groups > 1) && score == Ops::SoftmaxChosen) throw ConfigError("moe: a correction or groups do not go with weights from the chosen logits");
    for (const auto& c : children)
      if (c.first == "shared") shared = std::dynamic_pointer_cast<FeedForwardPart>(c.second);
    if (!shared && p.has("shared")) {
      const PartSpec sp = PartSpec::from_json(p.at("shared"));
      shared = std::dynamic_pointer_cast<FeedForwardPart>(build_part("ffn", sp, join(prefix, sp.name)));
    }
    if (shared && !shared->can_store()) throw ConfigError("moe: the shared feed-forward must be able to write its output apart from the residual");
  }
  std::vector<std::shared_ptr<Part>> children() const override {
    if (shared) return {shared};
    return {};
  }
  std::vector<std::string> child_slots() const override {
    if (shared) return {"shared"};
    return {};
  }
  const char* kind_name() const override { return "moe"; }
  bool reads_through_ops() const override { return true; }
  bool can_store() const override { return true; }
  std::string expert_name(int e, const char* t) const { return join(prefix, "e" + std::to_string(e) + "." + t); }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    TensorNeed up, down, router;
    up.shape = {intermediate, hidden};
    down.shape = {hidden, intermediate};
    router.shape = {(int64_t)experts, hidden};
    router.role = TensorNeed::Vector;      // held in 32-bit whatever the engine's dtype
    router.b = 0.1;
    for (int e = 0; e < experts; ++e) {
      if (gated) t.emplace_back(expert_name(e, "gate"), up);
      t.emplace_back(expert_name(e, "up"), up);
      t.emplace_back(expert_name(e, "down"), down);
    }
    t.emplace_back(n_router, router);
    if (corrected) {
      TensorNeed c;
      c.shape = {(int64_t)experts};
      c.role = TensorNeed::Vector;
      c.b = 0.3;
      t.emplace_back(n_correction, c);
    }
    return t;
  }
  void load(WeightSource& src) override {
    // the experts' matrices one under the other: a kernel finds expert e at row e * its rows (gated: an expert's gate rows
    // above its up rows)
    const int64_t up_rows = gated ? 2 * intermediate : intermediate;
    w_up = src.alloc(src.matrix_dtype, {(int64_t)experts * up_rows, hidden});
    w_down = src.alloc(src.matrix_dtype, {(int64_t)experts * hidden, intermediate});
    for (int e = 0; e < experts; ++e) {
      if (gated) src.fill(expert_name(e, "gate"), w_up.rows((int64_t)e * up_rows, intermediate));
      src.fill(expert_name(e, "up"), w_up.rows((int64_t)e * up_rows + (gated ? intermediate : 0), intermediate));
      src.fill(expert_name(e, "down"), w_down.rows((int64_t)e * hidden, hidden));
    }
    TensorNeed router;
    router.shape = {(int64_t)experts, hidden};
    router.role = TensorNeed::Vector;
    w_router = src.fetch(n_router, router);
    if (corrected) {
      TensorNeed c;
      c.shape = {(int64_t)experts};
      c.role = TensorNeed::Vector;
      correction = src.fetch(n_correction, c);
    }
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& y, Ops::GatheredRows* left) {
    const Tensor& rows = h.materialize(ctx.ops);
    const int64_t M = rows.shape[0];
    Tensor ids = ctx.buf("moe.ids", DType::I32, {M, (int64_t)top});
    Tensor wts = ctx.buf("moe.wts", DType::F32, {M, (int64_t)top});
    if (corrected || groups > 1 || weight_scale != 1.f || sum_floor != 0.f) {
      Ops::RouterGroups g;
      g.correction = correction;
      g.groups = groups;
      g.keep = keep;
      g.weight_scale = weight_scale;
      g.sum_floor = sum_floor;
      ctx.ops.moe_route(rows, w_router, ids, wts, top, score, renormalize, g);
    } else {
      ctx.ops.moe_route(rows, w_router, ids, wts, top, score, renormalize);
    }
    if (gated) ctx.ops.moe_experts_gated(rows, ids, wts, w_up, w_down, y, experts, act_kind, limit, alpha, ctx.ws, left);
    else ctx.ops.moe_experts(rows, ids, wts, w_up, w_down, y, experts, scale_input, ctx.ws, left);
  }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override {
    run(ctx, h, y, nullptr);
    if (shared) {      // the expert every token takes, added in 32-bit
      Tensor ys = ctx.buf("moe.shared", DType::F32, {y.shape[0], hidden});
      shared->forward_store(ctx, h, ys);
      ctx.ops.scaled_add(y, ys, Tensor(), Tensor(), Tensor());
    }
  }
  // the sum over a token's experts may be left to the norm that reads the result
  void forward_rows(StepContext& ctx, const Rows& h, const Tensor& y, Ops::GatheredRows& rows) override {
    if (shared) {
      forward_store(ctx, h, y);
      rows = Ops::GatheredRows();
      rows.t = y;
      return;
    }
    run(ctx, h, y, &rows);
    if (!rows.t.defined()) rows.t = y;
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor y = ctx.buf("moe.y", DType::F32, {x.shape[0], hidden});
    forward_store(ctx, h, y);
    ctx.ops.scaled_add(x, y, Tensor(), Tensor(), Tensor());
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w_up", w_up}, {"w_down", w_down}, {"w_router", w_router}}; }
  int64_t hidden = 0, intermediate = 0;
  int experts = 0, top = 0;
  Ops::RouterScore score = Ops::Sigmoid;
  bool renormalize = false, scale_input = true;
  bool gated = false;                      // `activation` glu_*: experts hold gate, up and down; the weight is on the output
  Ops::GatedAct act_kind = Ops::Silu;
  float limit = 0.f, alpha = 1.702f;       // glu_clamped: g = min(g, limit), u = clamp(u, -limit, limit), g sigmoid(alpha g) (u + 1)
  std::shared_ptr<FeedForwardPart> shared; // `shared`: a feed-forward every token takes, added to the experts' sum
  std::string n_router, n_correction;
  bool corrected = false;                  // `correction`: a vector added to the scores for the choice only (tensor prefix.correction)
  int groups = 0, keep = 0;                // `groups` {count, keep}: only experts of the best `keep` of `count` groups can be chosen
  float weight_scale = 1.f, sum_floor = 0.f;
  Tensor w_up, w_down, w_router, correction;
};

// Dynamic Tanh in the place of a norm: y = tanh(alpha x) * w + b, alpha one learned number, w and b vectors; no mean and no
// variance is taken.  Tensor names: `tensor` (default prefix + ".weight"), and that name with ".alpha" and ".b".
class DynamicTanh final : public NormPart {
 public:
  DynamicTanh(const std::string& prefix, const Json& p) : NormPart(prefix) {
    dim = param_int(p, "dim");
    name = tensor_name(p, "tensor", prefix, "weight");
    if (dim <= 0) throw ConfigError("dyt: dim must be positive");
  }
  const char* kind_name() const override { return "dyt"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed w, a, b;
    w.shape = b.shape = {dim};
    w.role = a.role = b.role = TensorNeed::Vector;
    w.a = 1.0;
    w.b = 0.1;
    a.a = 0.5;
    a.b = 0.05;
    b.b = 0.1;
    return {{name, w}, {name + ".alpha", a}, {name + ".b", b}};
  }
  void load(WeightSource& src) override {
    const auto t = tensors();
    weight = src.fetch(t[0].first, t[0].second);
    alpha = src.fetch(t[1].first, t[1].second);
    bias = src.fetch(t[2].first, t[2].second);
  }
  Rows forward(StepContext& ctx, const Tensor& x, const int* rows, int64_t n_rows, bool) override {
    const int64_t n = rows ? n_rows : x.shape[0];
    Rows r;
    r.t = ctx.buf("norm.out", ctx.act_dtype, {n, dim});
    ctx.ops.dyt(x, alpha, weight, bias, r.t, rows, n_rows);
    return r;
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}, {"alpha", alpha}, {"bias", bias}}; }
  int64_t dim = 0;
  std::string name;
  Tensor weight, alpha, bias;
};

// A gated feed-forward: down(act(gate h, up h)).  `activation` "silu": silu(g) u; "gelu_tanh": gelu(g) u with
// gelu(g) = g / 2 (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))); "clamped" (`limit`, `alpha` default 1.702):
// g = min(g, limit), u = clamp(u, -limit, limit), g sigmoid(alpha g) (u + 1).  `bias`: every projection has a bias (the
// tensor's name with ".b").  The first product leaves 32-bit sums of [gate | up] (one stacked weight), the activation is
// taken in 32-bit and rounded once.  Tensor names: prefix + ".gate", ".up", ".down" unless the parameters give them.
class GatedFFN final : public FeedForwardPart {
 public:
  GatedFFN(const std::string& prefix, const Json& p) : FeedForwardPart(prefix) {
    hidden = param_int(p, "hidden");
    intermediate = param_int(p, "intermediate");
    if (hidden <= 0 || intermediate <= 0) throw ConfigError("glu feed-forward: sizes must be positive");
    const std::string act = p.has("activation") ? p.at("activation").as_string() : "silu";
    if (act != "silu" && act != "clamped" && act != "gelu_tanh")
      throw ConfigError("glu feed-forward: activation '" + act + "' is not served (silu, clamped, gelu_tanh)");
    kind = act == "clamped" ? Ops::ClampedGlu : act == "gelu_tanh" ? Ops::GeluTanh : Ops::Silu;
    if (kind == Ops::ClampedGlu) {
      limit = (float)param_float(p, "limit");
      alpha = p.has("alpha") ? (float)param_float(p, "alpha") : 1.702f;
      if (!(limit > 0.f)) throw ConfigError("glu feed-forward: limit must be positive");
    }
    bias = p.has("bias") && p.at("bias").as_bool();
    n_gate = tensor_name(p, "gate", prefix, "gate");
    n_up = tensor_name(p, "up", prefix, "up");
    n_down = tensor_name(p, "down", prefix, "down");
  }
  const char* kind_name() const override { return "glu"; }
  bool reads_through_ops() const override { return true; }
  bool can_store() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed up, down, bu, bd;
    up.shape = {intermediate, hidden};
    down.shape = {hidden, intermediate};
    bu.shape = {intermediate};
    bd.shape = {hidden};
    bu.role = bd.role = TensorNeed::Vector;
    bu.b = bd.b = 0.2;
    std::vector<std::pair<std::string, TensorNeed>> t = {{n_gate, up}, {n_up, up}, {n_down, down}};
    if (bias) {
      t.emplace_back(n_gate + ".b", bu);
      t.emplace_back(n_up + ".b", bu);
      t.emplace_back(n_down + ".b", bd);
    }
    return t;
  }
  void load(WeightSource& src) override {
    w_gate_up = src.alloc(src.matrix_dtype, {2 * intermediate, hidden});
    src.fill(n_gate, w_gate_up.rows(0, intermediate));
    src.fill(n_up, w_gate_up.rows(intermediate, intermediate));
    TensorNeed down;
    down.shape = {hidden, intermediate};
    w_down = src.fetch(n_down, down);
    if (bias) {
      b_gate_up = src.alloc(DType::F32, {2 * intermediate});
      src.fill(n_gate + ".b", b_gate_up.rows(0, intermediate));
      src.fill(n_up + ".b", b_gate_up.rows(intermediate, intermediate));
      TensorNeed bd;
      bd.shape = {hidden};
      bd.role = TensorNeed::Vector;
      b_down = src.fetch(n_down + ".b", bd);
    }
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor z = ctx.buf("glu.z", DType::F32, {M, 2 * intermediate});
    ctx.ops.linear(h, w_gate_up, z, Ops::Store);
    Tensor y = ctx.buf("glu.y", ctx.act_dtype, {M, intermediate});
    ctx.ops.gated_act(z, b_gate_up, y, kind, limit, alpha);
    ctx.ops.linear(y, w_down, out, epi, false);
    if (bias) ctx.ops.add_row(out, b_down);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x, Ops::Add); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override { run(ctx, h, y, Ops::Store); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_gate_up", w_gate_up}, {"w_down", w_down}, {"b_gate_up", b_gate_up}, {"b_down", b_down}};
  }
  int64_t hidden = 0, intermediate = 0;
  Ops::GatedAct kind = Ops::Silu;
  float limit = 0.f, alpha = 1.702f;
  bool bias = false;
  std::string n_gate, n_up, n_down;
  Tensor w_gate_up, w_down, b_gate_up, b_down;
};

// Latent attention.  Per token the mixer keeps a latent c of `kv_rank` numbers and one rotated key part of `rot_dim` numbers
// that all heads share (paged rows [kv_rank + rot_dim]); keys and values are never kept per head.  q = W_q h, head by head
// [head_dim unrotated | rot_dim rotated]; W_dkv h has kv_rank + rot_dim rows: the first kv_rank, divided by their root mean
// square (eps) and multiplied by the vector `dkv.norm`, are c, the rest is the key part, rotated by the child `pos` as every
// head's last rot_dim query entries are.  A head's unrotated key is W_uk c (head_dim rows a head), its value W_uv c
// (v_head_dim rows a head); score = (q_plain . k_plain + q_rot . k_rot) scale; causal (`window` optional); the softmax's
// denominator also holds exp(sink_h), a learned number a head (`sink`, optional).  Then the output projection.
// Scores, softmax, the latent's norm and the rotation are 32-bit.  Tensor names: prefix + ".q", ".dkv", ".dkv.norm", ".uk",
// ".uv", ".sink", ".o".  Where the sizes allow (a latent of a multiple of 16 up to 512, latent and key part together a
// multiple of 8 up to 576, an unrotated query size that is a multiple of 8, a value size that is a multiple of 16) a page holds
// the latents a second time, transposed, and bfloat16 steps run on the matrix cores.
class LatentAttention final : public MixerPart {
 public:
  LatentAttention(const std::string& prefix, const Json& p, const PartChildren& children) : MixerPart(prefix) {
    hidden = param_int(p, "hidden");
    heads = (int)param_int(p, "heads");
    dim = (int)param_int(p, "head_dim");
    rot_dim = (int)param_int(p, "rot_dim");
    v_dim = p.has("v_head_dim") ? (int)param_int(p, "v_head_dim") : dim;
    rank = (int)param_int(p, "kv_rank");
    if (heads <= 0 || dim < 0 || rot_dim < 0 || dim + rot_dim <= 0 || v_dim <= 0 || rank <= 0)
      throw ConfigError("latent_attention: sizes must be positive");
    if (rank + rot_dim > 768 || dim > 1536)
      throw ConfigError("latent_attention: a latent of " + std::to_string(rank) + " + " + std::to_string(rot_dim) + " is not served (up to 768 together)");
    eps = (float)(p.has("eps") ? param_float(p, "eps") : 1e-6);
    scale = p.has("scale") ? (float)param_float(p, "scale") : (float)(1.0 / std::sqrt((double)(dim + rot_dim)));
    window = p.has("window") ? (int)param_int(p, "window") : 0;
    has_sink = !p.has("sink") || p.at("sink").as_bool();
    for (const auto& c : children)
      if (c.first == "pos") pos = std::dynamic_pointer_cast<PositionPart>(c.second);
    if (!pos && p.has("pos")) pos = std::dynamic_pointer_cast<PositionPart>(build_part("pos", PartSpec::from_json(p.at("pos")), prefix));
    nq = (int64_t)heads * (dim + rot_dim);
    nkv = (int64_t)rank + rot_dim;
    // sizes the matrix-core kernels take: the pages then hold the latents a second time, transposed
    transposed = dim % 8 == 0 && (dim + rot_dim) % 4 == 0 && rank % 16 == 0 && rank <= 512 && nkv % 8 == 0 && nkv <= 576 && v_dim % 16 == 0;
  }
  const char* kind_name() const override { return "latent_attention"; }
  bool can_store() const override { return true; }
  bool takes_lazy_norm() const override { return true; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    if (pos) return {pos};
    return {};
  }
  std::vector<std::string> child_slots() const override {
    if (pos) return {"pos"};
    return {};
  }
  std::string name(const char* t) const { return join(prefix, t); }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed q, dkv, nw, uk, uv, sk, o;
    q.shape = {nq, hidden};
    dkv.shape = {nkv, hidden};
    nw.shape = {(int64_t)rank};
    nw.role = TensorNeed::Vector;
    nw.a = 1.0;
    nw.b = 0.1;
    uk.shape = {(int64_t)heads * dim, (int64_t)rank};
    uv.shape = {(int64_t)heads * v_dim, (int64_t)rank};
    sk.shape = {(int64_t)heads};
    sk.role = TensorNeed::Vector;
    sk.b = 1.0;
    o.shape = {hidden, (int64_t)heads * v_dim};
    std::vector<std::pair<std::string, TensorNeed>> t = {{name("q"), q}, {name("dkv"), dkv}, {name("dkv.norm"), nw}, {name("uk"), uk},
                                                         {name("uv"), uv}};
    if (has_sink) t.emplace_back(name("sink"), sk);
    t.emplace_back(name("o"), o);
    return t;
  }
  void load(WeightSource& src) override {
    const auto t = tensors();
    w_in = src.alloc(src.matrix_dtype, {nq + nkv, hidden});      // queries above the down-projection: one product
    src.fill(name("q"), w_in.rows(0, nq));
    src.fill(name("dkv"), w_in.rows(nq, nkv));
    for (const auto& kv : t) {
      if (kv.first == name("dkv.norm")) norm_w = src.fetch(kv.first, kv.second);
      if (kv.first == name("uk")) w_uk = src.fetch(kv.first, kv.second);
      if (kv.first == name("uv")) w_uv = src.fetch(kv.first, kv.second);
      if (kv.first == name("sink")) sink = src.fetch(kv.first, kv.second);
      if (kv.first == name("o")) w_o = src.fetch(kv.first, kv.second);
    }
    if (transposed && w_uk.dtype == DType::BF16) w_uk_t = src.alloc(w_uk.dtype, {(int64_t)heads * rank, (int64_t)dim});
    uk_transposed = false;
  }
  void prepare(Ops& ops, int max_seq) override {
    (void)max_seq;
    if (w_uk_t.defined() && !uk_transposed) {
      ops.latent_transpose(w_uk, w_uk_t, heads);
      uk_transposed = true;
    }
  }
  bool has_cache() const override { return true; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::PagedRows;
    n.row_shape = {transposed ? nkv + rank : nkv};      // a page: its rows of nkv, then (transposed) the latents again as [rank][rows]
    n.window = window;
    return n;
  }
  // The lists of the matrix-core kernels: tiles of TILE_ROWS query rows over the entries of several tokens, and the rows
  // of single-token entries.  Every such mixer of a model asks for the same lists; the first one builds them.
  static constexpr int TILE_ROWS = 64;
  void plan(StepPlan& plan) const override {
    if (!transposed || plan.decode_only() || plan.has("lattn.tiles")) return;
    const auto& entries = plan.entries();
    size_t n_tiles = 0, n_rows = 0;
    for (const auto& e : entries) {
      if (e.n_tokens > 1) n_tiles += (size_t)(e.n_tokens + TILE_ROWS - 1) / TILE_ROWS;
      else ++n_rows;
    }
    int* tiles = plan.ints("lattn.tiles", 3 * n_tiles);
    int* rows = plan.ints("lattn.rows", n_rows);
    struct Tile { int keys, entry, row, n; };
    std::vector<Tile> order;
    order.reserve(n_tiles);
    size_t r = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
      const auto& e = entries[i];
      if (e.n_tokens == 1) {
        rows[r++] = e.row0;
        continue;
      }
      for (int q0 = 0; q0 < e.n_tokens; q0 += TILE_ROWS) {
        const int n = std::min(TILE_ROWS, e.n_tokens - q0);
        order.push_back({e.start + q0 + n, (int)i, e.row0 + q0, n});      // the keys its last row sees
      }
    }
    // from the tile that walks the most keys to the one that walks the fewest: the long ones start first
    std::stable_sort(order.begin(), order.end(), [](const Tile& a, const Tile& b) { return a.keys > b.keys; });
    for (size_t t = 0; t < order.size(); ++t) {
      tiles[3 * t] = order[t].entry;
      tiles[3 * t + 1] = order[t].row;
      tiles[3 * t + 2] = order[t].n;
    }
  }
  Ops::LatentLists lists(const StepContext& ctx) const {
    Ops::LatentLists l;
    l.entry_meta = ctx.entry_meta;
    // a captured graph serves every later step of its shape: what it launches is sized for the longest sequence
    l.context = ctx.plan && ctx.plan->sized_for_longest() ? ctx.plan->max_seq() : ctx.max_context;
    if (ctx.decode_only) {
      l.n_rows = (int)ctx.M;
      return l;
    }
    l.tiles = ctx.planned("lattn.tiles");
    l.n_tiles = (int)(ctx.planned_size("lattn.tiles") / 3);
    l.rows = ctx.planned("lattn.rows");
    l.n_rows = (int)ctx.planned_size("lattn.rows");
    return l;
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor proj = ctx.buf("latent.proj", DType::F32, {M, nq + nkv});
    ctx.ops.linear(h, w_in, proj, Ops::Store);
    const auto bound = ctx.binding(this);
    const Tensor pool = ctx.kv_pool(bound.first, bound.second);
    const Ops::CacheView view = ctx.cache_view(bound.first);
    Ops::Rotation rot;
    if (pos && !pos->fused(rot)) throw EngineError("latent_attention: the position encoding '" + std::string(pos->kind_name()) + "' has no fused form");
    ctx.ops.latent_prep(proj, (int)nq, norm_w, eps, rot, ctx.positions, ctx.slots, view, pool, heads, dim, rot_dim, rank);
    Tensor a = ctx.buf("latent.out", ctx.act_dtype, {M, (int64_t)heads * v_dim});
    const Ops::LatentLists l = lists(ctx);
    ctx.ops.latent_attention(proj, w_uk, w_uv, sink, pool, view, ctx.positions, ctx.slots, a, heads, dim, rot_dim, rank, v_dim, scale,
                             window, ctx.ws, w_uk_t, transposed && ctx.plan ? &l : nullptr);
    ctx.ops.linear(a, w_o, out, epi, false);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x, Ops::Add); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override { run(ctx, h, y, Ops::Store); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_in", w_in}, {"norm_w", norm_w}, {"w_uk", w_uk}, {"w_uv", w_uv}, {"sink", sink}, {"w_o", w_o}, {"w_uk_t", w_uk_t}};
  }
  int64_t hidden = 0, nq = 0, nkv = 0;
  int heads = 0, dim = 0, rot_dim = 0, v_dim = 0, rank = 0, window = 0;
  bool has_sink = true;
  bool transposed = false;      // the pages hold the latents transposed as well (sizes the matrix-core kernels take)
  bool uk_transposed = false;   // w_uk_t has been filled
  float eps = 1e-6f, scale = 1.f;
  std::shared_ptr<PositionPart> pos;
  Tensor w_in, norm_w, w_uk, w_uv, sink, w_o;
  Tensor w_uk_t;                // bfloat16: every head's W_uk transposed, [heads][rank][dim]
};

// Keeps a copy of the residual as it stands, under `name`, for a later block of the same step (the embedding's output that
// a looped run of layers mixes in again before each pass).
class KeepBlock final : public BlockPart {
 public:
  KeepBlock(const std::string& prefix, const Json& p) : BlockPart(prefix) {
    name = p.has("name") ? p.at("name").as_string() : std::string("kept");
  }
  const char* kind_name() const override { return "keep"; }
  void forward(StepContext& ctx, const Tensor& x) override {
    ctx.ops.flush();
    Tensor k = ctx.buf("kept." + name, DType::F32, {x.shape[0], x.shape[1]});
    ctx.ops.fill_zero(k.data, k.bytes());
    ctx.ops.scaled_add(k, x, Tensor(), Tensor(), Tensor());
  }
  std::string name;
};

// x <- W [x; kept]: the residual and the stream a `keep` block left under `from`, side by side through one learned matrix
// [dim, 2 dim] (the residual's columns first).  `tensor`: the matrix's name; several such blocks share it.
class MixInBlock final : public BlockPart {
 public:
  MixInBlock(const std::string& prefix, const Json& p) : BlockPart(prefix) {
    dim = param_int(p, "dim");
    from = p.has("from") ? p.at("from").as_string() : std::string("kept");
    name = tensor_name(p, "tensor", prefix, "weight");
  }
  const char* kind_name() const override { return "mix_in"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    n.shape = {dim, 2 * dim};
    return {{name, n}};
  }
  void load(WeightSource& src) override { w = src.fetch(name, tensors()[0].second); }
  void forward(StepContext& ctx, const Tensor& x) override {
    ctx.ops.flush();
    const int64_t M = x.shape[0];
    const Tensor kept = ctx.buf("kept." + from, DType::F32, {M, dim});
    Tensor both = ctx.buf("mix_in.rows", ctx.act_dtype, {M, 2 * dim});
    ctx.ops.concat_round(x, kept, both);
    ctx.ops.linear(both, w, x, Ops::Store);
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"w", w}}; }
  int64_t dim = 0;
  std::string from, name;
  Tensor w;
};

// x += norm1(mixer(x)); x += norm2(ffn(x)).  The sublayers read the residual itself (rounded to the compute dtype where
// that is not 32-bit) and the norms are taken on what they return, in 32-bit, straight into the residual.  A layer may
// have no feed-forward (then no norm2 either).
class PostNormBlock final : public BlockPart {
 public:
  PostNormBlock(const std::string& prefix, const PartChildren& c) : BlockPart(prefix) {
    for (const auto& kv : c) {
      if (kv.first == "norm1") norm1 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "mixer") mixer = std::dynamic_pointer_cast<MixerPart>(kv.second);
      if (kv.first == "norm2") norm2 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "ffn") ffn = std::dynamic_pointer_cast<FeedForwardPart>(kv.second);
    }
    if (!norm1 || !mixer) throw ConfigError("block 'post_norm' needs norm1 and mixer parts (norm2 and ffn are optional)");
    if ((ffn != nullptr) != (norm2 != nullptr)) throw ConfigError("block 'post_norm': norm2 and ffn come together or not at all");
    if (!norm1->can_add() || (norm2 && !norm2->can_add())) throw ConfigError("block 'post_norm': its norms must be able to write into the residual");
    if (!mixer->can_store() || (ffn && !ffn->can_store()))
      throw ConfigError("block 'post_norm': its mixer and feed-forward must be able to write their output apart from the residual");
  }
  const char* kind_name() const override { return "post_norm"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    std::vector<std::shared_ptr<Part>> v = {norm1, mixer};
    if (ffn) {
      v.push_back(norm2);
      v.push_back(ffn);
    }
    return v;
  }
  std::vector<std::string> child_slots() const override {
    std::vector<std::string> v = {"norm1", "mixer"};
    if (ffn) {
      v.push_back("norm2");
      v.push_back("ffn");
    }
    return v;
  }
  // the rows a sublayer reads: the residual itself in a 32-bit engine, else its rounding
  Rows input(StepContext& ctx, const Tensor& x) {
    ctx.ops.flush();
    Rows h;
    if (ctx.act_dtype == DType::F32) {
      h.t = x;
      return h;
    }
    h.t = ctx.buf("post_norm.h", ctx.act_dtype, {x.shape[0], x.shape[1]});
    ctx.ops.round_rows(x, h.t);
    return h;
  }
  void forward(StepContext& ctx, const Tensor& x) override {
    Tensor y = ctx.buf("post_norm.y", DType::F32, {x.shape[0], x.shape[1]});
    mixer->forward_store(ctx, input(ctx, x), y);
    if (!ffn) {
      norm1->forward_add(ctx, y, x, true);
      return;
    }
    // the kernel that adds the normed rows also leaves the rounding of the new residual for the feed-forward
    Rows h;
    if (ctx.act_dtype == DType::F32) {
      norm1->forward_add(ctx, y, x, true);
      h.t = x;
    } else {
      h.t = ctx.buf("post_norm.h", ctx.act_dtype, {x.shape[0], x.shape[1]});
      norm1->forward_add(ctx, y, x, true, nullptr, 0, &h.t);
    }
    Ops::GatheredRows rows;
    ffn->forward_rows(ctx, h, y, rows);
    norm2->forward_add(ctx, rows.t, x, true, rows.gather, rows.n_gather);
  }
  std::shared_ptr<NormPart> norm1, norm2;
  std::shared_ptr<MixerPart> mixer;
  std::shared_ptr<FeedForwardPart> ffn;
};

// A layer norm with a gain and no bias: y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w, in 32-bit, rounded once.
// `tensor`: the weight's name in the checkpoint (default: prefix + ".weight").  It can norm 32-bit rows in place (an embedding's
// rows) and take a weighted sum of several streams as its input without that sum being formed.
class LayerNorm final : public NormPart {
 public:
  LayerNorm(const std::string& prefix, const Json& p) : NormPart(prefix) {
    dim = param_int(p, "dim");
    eps = (float)param_float(p, "eps");
    name = tensor_name(p, "tensor", prefix, "weight");
    if (dim <= 0 || dim > 16384) throw ConfigError("layernorm: a width of " + std::to_string(dim) + " is not served (1 to 16384)");
  }
  const char* kind_name() const override { return "layernorm"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed n;
    n.shape = {dim};
    n.role = TensorNeed::Vector;
    n.a = 1.0;
    n.b = 0.1;
    return {{name, n}};
  }
  void load(WeightSource& src) override { weight = src.fetch(name, tensors()[0].second); }
  Rows forward(StepContext& ctx, const Tensor& x, const int* rows, int64_t n_rows, bool) override {
    Rows r;
    r.t = ctx.buf("norm.out", ctx.act_dtype, {rows ? n_rows : x.shape[0], dim});
    ctx.ops.layernorm(x, weight, eps, r.t, rows, n_rows);
    return r;
  }
  bool can_add() const override { return true; }
  void forward_add(StepContext& ctx, const Tensor& y, const Tensor& x, bool accumulate, const int* gather, int n_gather,
                   const Tensor* rounded) override {
    if (accumulate || gather || n_gather > 1 || rounded) throw EngineError("layernorm: it norms 32-bit rows in place, nothing else");
    ctx.ops.layernorm(y, weight, eps, x);
  }
  bool can_mix() const override { return true; }
  Rows forward_mixed(StepContext& ctx, const Tensor& streams, const Tensor& coef) override {
    Rows r;
    r.t = ctx.buf("norm.out", ctx.act_dtype, {streams.shape[1], dim});
    ctx.ops.layernorm_mixed(streams, coef, weight, eps, r.t);
    return r;
  }
  bool mixed_form(StepContext& ctx, int64_t M, Tensor& w, float& e, Rows& rows) override {
    w = weight;
    e = eps;
    rows = Rows();
    rows.t = ctx.buf("norm.out", ctx.act_dtype, {M, dim});
    return true;
  }
  std::vector<std::pair<std::string, Tensor>> held() const override { return {{"weight", weight}}; }
  int64_t dim = 0;
  float eps = 1e-6f;
  std::string name;
  Tensor weight;
};

// The residual in `streams` copies (hyper-connections).  "hyper_spread" makes every stream a copy of the residual as the
// embedding left it; a "hyper" layer works on the streams; "hyper_sum" puts their sum back into the residual for the final
// norm.  The streams of a step lie in the workspace under one name, f32 [streams, M, dim].
static Tensor hyper_streams(StepContext& ctx, int64_t streams, int64_t M, int64_t dim) {
  return ctx.buf("hyper.streams", DType::F32, {streams, M, dim});
}
// A layer may leave its last write into the streams as a note (`defer_write`): tensors (mix, back, y, y2 or undefined), numbers
// (f1, f2).  The next layer's first read takes it in (one pass over the streams instead of two); whoever else needs the streams
// complete does the write first.
static const char* const HYPER_PENDING = "hyper.pending";
static bool hyper_take_pending(StepContext& ctx, StepContext::Note& note) {
  auto it = ctx.notes.find(HYPER_PENDING);
  if (it == ctx.notes.end()) return false;
  note = std::move(it->second);
  ctx.notes.erase(it);
  return true;
}
static void hyper_flush(StepContext& ctx, const Tensor& xs) {
  StepContext::Note n;
  if (hyper_take_pending(ctx, n))
    ctx.ops.hyper_write(xs, n.tensors[0], n.tensors[1], n.tensors[2], n.tensors[3], (float)n.numbers[0], (float)n.numbers[1]);
}
class HyperSpreadBlock final : public BlockPart {
 public:
  HyperSpreadBlock(const std::string& prefix, const Json& p) : BlockPart(prefix), streams(param_int(p, "streams")), dim(param_int(p, "dim")) {}
  const char* kind_name() const override { return "hyper_spread"; }
  void forward(StepContext& ctx, const Tensor& x) override {
    ctx.ops.flush();
    ctx.notes.erase(HYPER_PENDING);
    ctx.ops.hyper_spread(x, hyper_streams(ctx, streams, x.shape[0], dim));
  }
  int64_t streams, dim;
};
class HyperSumBlock final : public BlockPart {
 public:
  HyperSumBlock(const std::string& prefix, const Json& p) : BlockPart(prefix), streams(param_int(p, "streams")), dim(param_int(p, "dim")) {}
  const char* kind_name() const override { return "hyper_sum"; }
  void forward(StepContext& ctx, const Tensor& x) override {
    ctx.ops.flush();
    const Tensor xs = hyper_streams(ctx, streams, x.shape[0], dim);
    hyper_flush(ctx, xs);
    ctx.ops.hyper_combine(xs, Tensor(), x);
  }
  int64_t streams, dim;
};

// A layer on a residual of `streams` copies x_1 .. x_S.  Sublayer q (1: the mixer, 2: the feed-forward, which may be absent)
// reads u = sum_s in_q[s] x_s through its norm, and its output y goes back into all streams at once:
// x_t <- sum_s mix_q[s, t] x_s + out_q[t] y (mix indexed [from, to]).  Tensors: prefix + ".hc<q>.in" [S], ".hc<q>.out" [S],
// ".hc<q>.mix" [S, S], held in 32-bit.  A norm that can take the weighted sum in does (no u is written); the sublayers write
// apart from the residual.  The mixer's write takes the feed-forward's read in; with `defer_write` the layer's last write is left
// as a note for the next layer's first read (or for `hyper_sum`), which takes it in the same way.
class HyperBlock final : public BlockPart {
 public:
  HyperBlock(const std::string& prefix, const Json& p, const PartChildren& c) : BlockPart(prefix) {
    for (const auto& kv : c) {
      if (kv.first == "norm1") norm1 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "mixer") mixer = std::dynamic_pointer_cast<MixerPart>(kv.second);
      if (kv.first == "norm2") norm2 = std::dynamic_pointer_cast<NormPart>(kv.second);
      if (kv.first == "ffn") ffn = std::dynamic_pointer_cast<FeedForwardPart>(kv.second);
    }
    if (!norm1 || !mixer) throw ConfigError("block 'hyper' needs norm1 and mixer parts (norm2 and ffn are optional)");
    if ((ffn != nullptr) != (norm2 != nullptr)) throw ConfigError("block 'hyper': norm2 and ffn come together or not at all");
    if (!mixer->can_store() || (ffn && !ffn->can_store()))
      throw ConfigError("block 'hyper': its mixer and feed-forward must be able to write their output apart from the residual");
    streams = param_int(p, "streams");
    dim = param_int(p, "dim");
    defer_write = p.has("defer_write") && p.at("defer_write").as_bool();
    if (streams < 1 || streams > 16) throw ConfigError("block 'hyper': " + std::to_string(streams) + " streams are not served (1 to 16)");
  }
  const char* kind_name() const override { return "hyper"; }
  bool reads_through_ops() const override { return true; }
  std::vector<std::shared_ptr<Part>> children() const override {
    std::vector<std::shared_ptr<Part>> v = {norm1, mixer};
    if (ffn) {
      v.push_back(norm2);
      v.push_back(ffn);
    }
    return v;
  }
  std::vector<std::string> child_slots() const override {
    std::vector<std::string> v = {"norm1", "mixer"};
    if (ffn) {
      v.push_back("norm2");
      v.push_back("ffn");
    }
    return v;
  }
  std::string name(int q, const char* t) const { return join(prefix, "hc" + std::to_string(q) + "." + t); }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    std::vector<std::pair<std::string, TensorNeed>> t;
    for (int q = 1; q <= (ffn ? 2 : 1); ++q) {
      TensorNeed in, out, mix;
      in.shape = out.shape = {streams};
      mix.shape = {streams, streams};
      in.role = out.role = mix.role = TensorNeed::Vector;
      in.a = 1.0 / (double)streams;
      in.b = 0.2;
      out.a = 1.0;
      out.b = 0.3;
      mix.a = 1.0 / (double)streams;
      mix.b = 0.3;
      t.emplace_back(name(q, "in"), in);
      t.emplace_back(name(q, "out"), out);
      t.emplace_back(name(q, "mix"), mix);
    }
    return t;
  }
  void load(WeightSource& src) override {
    const auto t = tensors();
    for (int q = 0; q < (ffn ? 2 : 1); ++q) {
      w_in[q] = src.fetch(t[3 * q].first, t[3 * q].second);
      w_out[q] = src.fetch(t[3 * q + 1].first, t[3 * q + 1].second);
      w_mix[q] = src.fetch(t[3 * q + 2].first, t[3 * q + 2].second);
    }
  }
  Rows read(StepContext& ctx, NormPart& norm, const Tensor& xs, const Tensor& coef) {
    if (norm.can_mix()) return norm.forward_mixed(ctx, xs, coef);
    Tensor u = ctx.buf("hyper.u", DType::F32, {xs.shape[1], dim});
    ctx.ops.hyper_combine(xs, coef, u);
    return norm.forward(ctx, u);
  }
  void forward(StepContext& ctx, const Tensor& x) override {
    const int64_t M = x.shape[0];
    const Tensor xs = hyper_streams(ctx, streams, M, dim);
    Tensor y = ctx.buf("hyper.y", DType::F32, {M, dim}), y2;
    // the write the layer before left undone goes into this layer's first read, where the norm has a form for that
    Rows h;
    StepContext::Note left;
    Tensor w1;
    float eps1 = 0.f;
    if (hyper_take_pending(ctx, left)) {
      if (norm1->mixed_form(ctx, M, w1, eps1, h)) {
        ctx.ops.hyper_write(xs, left.tensors[0], left.tensors[1], left.tensors[2], left.tensors[3], (float)left.numbers[0],
                            (float)left.numbers[1], w_in[0], w1, eps1, h.t);
      } else {
        ctx.ops.hyper_write(xs, left.tensors[0], left.tensors[1], left.tensors[2], left.tensors[3], (float)left.numbers[0],
                            (float)left.numbers[1]);
        h = read(ctx, *norm1, xs, w_in[0]);
      }
    } else {
      h = read(ctx, *norm1, xs, w_in[0]);
    }
    float f1 = 1.f, f2 = 1.f;
    if (mixer->leaves_pair()) {      // two branches left apart: the write adds them on its way
      y2 = ctx.buf("hyper.y2", DType::F32, {M, dim});
      mixer->forward_pair(ctx, h, y, y2, f1, f2);
    } else {
      mixer->forward_store(ctx, h, y);
    }
    if (!ffn) {
      if (defer_write) ctx.notes[HYPER_PENDING] = StepContext::Note{{w_mix[0], w_out[0], y, y2}, {f1, f2}};
      else ctx.ops.hyper_write(xs, w_mix[0], w_out[0], y, y2, f1, f2);
      return;
    }
    // the mixer's write and the feed-forward's read in one pass over the streams, where the norm has a form for that
    Tensor nw;
    float neps = 0.f;
    Rows h2;
    if (norm2->mixed_form(ctx, M, nw, neps, h2)) {
      ctx.ops.hyper_write(xs, w_mix[0], w_out[0], y, y2, f1, f2, w_in[1], nw, neps, h2.t);
    } else {
      ctx.ops.hyper_write(xs, w_mix[0], w_out[0], y, y2, f1, f2);
      h2 = read(ctx, *norm2, xs, w_in[1]);
    }
    ffn->forward_store(ctx, h2, y);
    if (defer_write) ctx.notes[HYPER_PENDING] = StepContext::Note{{w_mix[1], w_out[1], y, Tensor()}, {1.0, 1.0}};
    else ctx.ops.hyper_write(xs, w_mix[1], w_out[1], y);
  }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"in1", w_in[0]}, {"out1", w_out[0]}, {"mix1", w_mix[0]}, {"in2", w_in[1]}, {"out2", w_out[1]}, {"mix2", w_mix[1]}};
  }
  std::shared_ptr<NormPart> norm1, norm2;
  std::shared_ptr<MixerPart> mixer;
  std::shared_ptr<FeedForwardPart> ffn;
  int64_t streams = 1, dim = 0;
  bool defer_write = false;     // `defer_write`: the layer's last write is left to the next reader of the streams (a `hyper` layer or `hyper_sum`)
  Tensor w_in[2], w_out[2], w_mix[2];
};

// Linear attention with a fixed decay per head.  q = silu(W_q h), k = silu(W_k h) (heads x head_dim), v = silu(W_v h)
// (heads x v_head_dim); per head S_t = decay_h S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, no other scale; the heads side by side
// are divided by their root mean square over the whole row (eps), multiplied by the vector `norm` and by sigmoid(W_g h), and W_o
// maps them back.  q, k, v and the gate come from one product with the stacked weight [q; k; v; g].  S (heads x head_dim x
// v_head_dim) is per-request state in 32-bit, zero at admission; activations, state, outputs and the norm are 32-bit.
// `decay`: the heads' factors.  Tensor names: prefix + ".q", ".k", ".v", ".g", ".o", ".norm".
class DecayAttention final : public MixerPart {
 public:
  DecayAttention(const std::string& prefix, const Json& p) : MixerPart(prefix) {
    hidden = param_int(p, "hidden");
    heads = (int)param_int(p, "heads");
    dk = (int)param_int(p, "head_dim");
    dv = p.has("v_head_dim") ? (int)param_int(p, "v_head_dim") : dk;
    eps = (float)param_float(p, "eps");
    if (heads <= 0 || dk <= 0 || dv <= 0 || hidden <= 0) throw ConfigError("decay_attention: sizes must be positive");
    if (dk > 256 || dv > 256) throw ConfigError("decay_attention: a state of " + std::to_string(dk) + " x " + std::to_string(dv) + " a head is not served (up to 256 x 256)");
    const Json* d = p.find("decay");
    if (!d || d->type() != Json::Array || (int)d->size() != heads) throw ConfigError("decay_attention: 'decay' must list one factor a head");
    for (const Json& v : d->items()) {
      if (!v.is_number()) throw ConfigError("decay_attention: 'decay' must hold numbers");
      decay.push_back((float)v.as_double());
    }
    nq = (int64_t)heads * dk;
    nv = (int64_t)heads * dv;
    width = 2 * nq + 2 * nv;
  }
  const char* kind_name() const override { return "decay_attention"; }
  bool takes_lazy_norm() const override { return true; }
  bool reads_through_ops() const override { return true; }
  bool can_store() const override { return true; }
  std::string name(const char* t) const { return join(prefix, t); }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override {
    TensorNeed qk, v, o, nw;
    qk.shape = {nq, hidden};
    v.shape = {nv, hidden};
    o.shape = {hidden, nv};
    nw.shape = {nv};
    nw.role = TensorNeed::Vector;
    nw.a = 1.0;
    nw.b = 0.1;
    return {{name("q"), qk}, {name("k"), qk}, {name("v"), v}, {name("g"), v}, {name("o"), o}, {name("norm"), nw}};
  }
  void load(WeightSource& src) override {
    w_in = src.alloc(src.matrix_dtype, {width, hidden});
    src.fill(name("q"), w_in.rows(0, nq));
    src.fill(name("k"), w_in.rows(nq, nq));
    src.fill(name("v"), w_in.rows(2 * nq, nv));
    src.fill(name("g"), w_in.rows(2 * nq + nv, nv));
    const auto t = tensors();
    w_o = src.fetch(t[4].first, t[4].second);
    norm_w = src.fetch(t[5].first, t[5].second);
    w_decay = src.alloc(DType::F32, {(int64_t)heads});
    put_floats(w_decay, decay, src.to_host);
  }
  static void put_floats(const Tensor& dst, const std::vector<float>& values, bool on_host);
  bool has_cache() const override { return true; }
  CacheNeed cache_need() const override {
    CacheNeed n;
    n.kind = CacheNeed::State;
    n.state_shape = {heads, (int64_t)dk * dv};
    return n;
  }
  // A step with a long portion: every entry's tokens in chunks of CHUNK that run side by side (the state is carried from chunk
  // to chunk element by element), from CHUNK_FROM tokens on.  The lists are the same for every such mixer of the model; the
  // first one builds them.
  static constexpr int CHUNK = 64, CHUNK_FROM = 128;
  void plan(StepPlan& plan) const override {
    if (plan.decode_only() || plan.has("decay.chunks")) return;
    const auto& entries = plan.entries();
    int longest = 0;
    size_t n_chunks = 0;
    for (const auto& e : entries) {
      longest = std::max(longest, e.n_tokens);
      n_chunks += (size_t)(e.n_tokens + CHUNK - 1) / CHUNK;
    }
    if (longest < CHUNK_FROM) return;
    int* chunks = plan.ints("decay.chunks", 4 * n_chunks);
    int* spans = plan.ints("decay.spans", 2 * entries.size());
    int c = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
      const auto& e = entries[i];
      const int n = (e.n_tokens + CHUNK - 1) / CHUNK;
      spans[2 * i] = c;
      spans[2 * i + 1] = n;
      for (int k = 0; k < n; ++k, ++c) {
        chunks[4 * c] = (int)i;
        chunks[4 * c + 1] = e.row0 + k * CHUNK;
        chunks[4 * c + 2] = std::min(CHUNK, e.n_tokens - k * CHUNK);
        chunks[4 * c + 3] = (k == 0 ? 1 : 0) | (k == n - 1 ? 2 : 0);
      }
    }
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& out, Ops::Epilogue epi) {
    const int64_t M = h.t.shape[0];
    Tensor proj = ctx.buf("decay.proj", DType::F32, {M, width});
    ctx.ops.linear(h, w_in, proj, Ops::Store);
    const auto bound = ctx.binding(this);
    const Tensor state = ctx.state(bound.first, bound.second);
    Tensor o = ctx.buf("decay.o", DType::F32, {M, nv});
    Ops::QkvColumns cols;
    cols.q = 0;
    cols.k = (int)nq;
    cols.v = (int)(2 * nq);
    ctx.ops.decay_scan(proj, cols, w_decay, state, ctx.entry_meta, (int)ctx.entries.size(), o, heads, dk, dv, ctx.planned("decay.chunks"),
                       (int)(ctx.planned_size("decay.chunks") / 4), ctx.planned("decay.spans"), &ctx.ws);
    Tensor a = ctx.buf("decay.gated", ctx.act_dtype, {M, nv});
    ctx.ops.gated_row_norm(o, proj, (int)(2 * nq + nv), norm_w, eps, a);
    ctx.ops.linear(a, w_o, out, epi, epi == Ops::Add);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x, Ops::Add); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override { run(ctx, h, y, Ops::Store); }
  std::vector<std::pair<std::string, Tensor>> held() const override {
    return {{"w_in", w_in}, {"w_o", w_o}, {"norm_w", norm_w}, {"decay", w_decay}};
  }
  int64_t hidden = 0, nq = 0, nv = 0, width = 0;
  int heads = 0, dk = 0, dv = 0;
  float eps = 1e-6f;
  std::vector<float> decay;
  Tensor w_in, w_o, norm_w, w_decay;
};

// Two mixers side by side on the same input: y = left_scale * left(h) + right_scale * right(h), added in 32-bit.  `left`,
// `right`: the two mixers as parts ({"kind", "params", "name"}; the name follows this part's prefix); each keeps its own cache
// or state.
class SumMixer final : public MixerPart {
 public:
  SumMixer(const std::string& prefix, const Json& p, const PartChildren& children) : MixerPart(prefix) {
    dim = param_int(p, "hidden");
    left_scale = (float)param_float(p, "left_scale");
    right_scale = (float)param_float(p, "right_scale");
    for (const auto& c : children) {
      if (c.first == "left") left = std::dynamic_pointer_cast<MixerPart>(c.second);
      if (c.first == "right") right = std::dynamic_pointer_cast<MixerPart>(c.second);
    }
    auto build = [&](const char* key) {
      const PartSpec sp = PartSpec::from_json(p.at(key));
      return std::dynamic_pointer_cast<MixerPart>(build_part("mixer", sp, join(prefix, sp.name)));
    };
    if (!left && p.has("left")) left = build("left");
    if (!right && p.has("right")) right = build("right");
    if (!left || !right) throw ConfigError("mixer 'sum' needs a left and a right mixer");
    if (!left->can_store() || !right->can_store()) throw ConfigError("mixer 'sum': both mixers must be able to write their output apart from the residual");
  }
  const char* kind_name() const override { return "sum"; }
  bool can_store() const override { return true; }
  bool reads_through_ops() const override { return left->reads_through_ops() && right->reads_through_ops(); }
  std::vector<std::shared_ptr<Part>> children() const override { return {left, right}; }
  std::vector<std::string> child_slots() const override { return {"left", "right"}; }
  void load(WeightSource& src) override {
    s_left = src.alloc(DType::F32, {dim});
    s_right = src.alloc(DType::F32, {dim});
    DecayAttention::put_floats(s_left, std::vector<float>((size_t)dim, left_scale), src.to_host);
    DecayAttention::put_floats(s_right, std::vector<float>((size_t)dim, right_scale), src.to_host);
  }
  void run(StepContext& ctx, const Rows& h, const Tensor& x) {
    const int64_t M = h.t.shape[0];
    Tensor y1 = ctx.buf("sum.left", DType::F32, {M, dim}), y2 = ctx.buf("sum.right", DType::F32, {M, dim});
    left->forward_store(ctx, h, y1);
    right->forward_store(ctx, h, y2);
    ctx.ops.scaled_add(x, y1, s_left, y2, s_right);
  }
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override { run(ctx, h, x); }
  void forward_store(StepContext& ctx, const Rows& h, const Tensor& y) override {
    ctx.ops.fill_zero(y.data, y.bytes());
    run(ctx, h, y);
  }
  bool leaves_pair() const override { return true; }
  void forward_pair(StepContext& ctx, const Rows& h, const Tensor& y1, const Tensor& y2, float& f1, float& f2) override {
    left->forward_store(ctx, h, y1);
    right->forward_store(ctx, h, y2);
    f1 = left_scale;
    f2 = right_scale;
  }
  std::shared_ptr<MixerPart> left, right;
  int64_t dim = 0;
  float left_scale = 1.f, right_scale = 1.f;
  Tensor s_left, s_right;      // the factors spread over a row: what the kernel that adds two scaled branches takes
};

void register_builtin_parts() {
  register_part("norm", "layernorm", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<LayerNorm>(prefix, p);
  });
  register_part("block", "hyper_spread",
                [](const std::string& prefix, const Json& p, const PartChildren&) { return std::make_shared<HyperSpreadBlock>(prefix, p); });
  register_part("block", "hyper_sum",
                [](const std::string& prefix, const Json& p, const PartChildren&) { return std::make_shared<HyperSumBlock>(prefix, p); });
  register_part("block", "hyper",
                [](const std::string& prefix, const Json& p, const PartChildren& c) { return std::make_shared<HyperBlock>(prefix, p, c); },
                {{"norm1", "norm"}, {"mixer", "mixer"}, {"norm2", "norm?"}, {"ffn", "ffn?"}});
  register_part("mixer", "decay_attention", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<DecayAttention>(prefix, p);
  });
  register_part("mixer", "sum", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<SumMixer>(prefix, p, c);
  });
  register_part("pos", "rope_partial", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<RotaryPartial>(prefix, p);
  });
  register_part("filter", "short_conv", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<ShortConv>(prefix, p);
  });
  register_part("mixer", "diff_attention", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<DiffAttention>(prefix, p, c);
  });
  register_part("ffn", "moe", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<MoE>(prefix, p, c);
  });
  register_part("norm", "dyt", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<DynamicTanh>(prefix, p);
  });
  register_part("ffn", "glu", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<GatedFFN>(prefix, p);
  });
  register_part("mixer", "latent_attention", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<LatentAttention>(prefix, p, c);
  });
  register_part("block", "keep",
                [](const std::string& prefix, const Json& p, const PartChildren&) { return std::make_shared<KeepBlock>(prefix, p); });
  register_part("block", "mix_in",
                [](const std::string& prefix, const Json& p, const PartChildren&) { return std::make_shared<MixInBlock>(prefix, p); });
  register_part("block", "post_norm",
                [](const std::string& prefix, const Json&, const PartChildren& c) { return std::make_shared<PostNormBlock>(prefix, c); },
                {{"norm1", "norm"}, {"mixer", "mixer"}, {"norm2", "norm?"}, {"ffn", "ffn?"}});
  register_part("embedding", "table", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<Embedding>(prefix, p, c);
  });
  register_part("head", "linear", [](const std::string& prefix, const Json& p, const PartChildren&) {
    const Json* t = p.find("tied");
    const int tied = (!t || t->is_null()) ? -1 : (t->as_bool() ? 1 : 0);
    return std::make_shared<LMHead>(prefix, param_int(p, "vocab"), param_int(p, "dim"), tied,
                                    p.has("tied_to") ? p.at("tied_to").as_string() : std::string(),
                                    tensor_name(p, "tensor", prefix, "weight"), p.has("scale") ? param_float(p, "scale") : 1.0);
  });
  register_part("norm", "rmsnorm", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<RMSNorm>(prefix, param_int(p, "dim"), param_float(p, "eps"), p.has("scalar") && p.at("scalar").as_bool(),
                                     p.has("tensor") ? p.at("tensor").as_string() : std::string(),
                                     p.has("one_plus") && p.at("one_plus").as_bool());
  });
  register_part("pos", "rope_neox", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<RotaryNeox>(prefix, param_int(p, "head_dim"), param_float(p, "theta"));
  });
  register_part("pos", "sinusoidal", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<Sinusoidal>(prefix, param_int(p, "dim"), p.has("base") ? param_float(p, "base") : 10000.0);
  });
  register_part("ffn", "dense", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<DenseFFN>(prefix, p);
  });
  register_part("mixer", "mlstm", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<MLSTM>(prefix, p);
  });
  register_part("block", "parallel",
                [](const std::string& prefix, const Json& p, const PartChildren& c) { return std::make_shared<ParallelBlock>(prefix, p, c); },
                {{"norm1", "norm"}, {"mixer", "mixer"}, {"ffn", "ffn?"}});
  register_part("block", "add_vector",
                [](const std::string& prefix, const Json& p, const PartChildren&) { return std::make_shared<AddVectorBlock>(prefix, p); });
  register_part("ffn", "swiglu", [](const std::string& prefix, const Json& p, const PartChildren&) {
    return std::make_shared<SwiGLU>(prefix, param_int(p, "hidden"), param_int(p, "intermediate"));
  });
  register_part("mixer", "attention", [](const std::string& prefix, const Json& p, const PartChildren& c) {
    return std::make_shared<Attention>(prefix, p, c);
  });
  register_part("block", "pre_norm",
                [](const std::string& prefix, const Json&, const PartChildren& c) { return std::make_shared<PreNormBlock>(prefix, c); },
                {{"norm1", "norm"}, {"mixer", "mixer"}, {"norm2", "norm?"}, {"ffn", "ffn?"}});
}

// --------------------------------------------------------------------------------- foreign parts
ForeignCalls g_foreign;
thread_local std::string g_foreign_error;

struct ForeignInfo {
  std::vector<std::pair<std::string, TensorNeed>> tensors;
  bool has_cache = false;
  CacheNeed cache;
  bool takes_lazy = false;
};

ForeignInfo read_description(const Json& d) {
  ForeignInfo info;
  if (const Json* ts = d.find("tensors"))
    for (const auto& kv : ts->members()) {
      TensorNeed n;
      for (const Json& s : kv.second.at("shape").items()) n.shape.push_back(s.as_int());
      const std::string role = kv.second.has("role") ? kv.second.at("role").as_string() : "matrix";
      n.role = role == "vector" ? TensorNeed::Vector : role == "table" ? TensorNeed::Table : TensorNeed::Matrix;
      if (kv.second.has("init")) n.init = kv.second.at("init").as_string();
      if (kv.second.has("a")) n.a = kv.second.at("a").as_double();
      if (kv.second.has("b")) n.b = kv.second.at("b").as_double();
      n.optional = kv.second.has("optional") && kv.second.at("optional").as_bool();
      info.tensors.emplace_back(kv.first, n);
    }
  if (d.has("cache_need")) {
    const Json& c = d.at("cache_need");
    info.has_cache = true;
    if (c.at("kind").as_string() == "state") {
      info.cache.kind = CacheNeed::State;
      for (const Json& s : c.at("shape").items()) info.cache.state_shape.push_back(s.as_int());
    } else if (c.at("kind").as_string() == "paged_rows") {
      info.cache.kind = CacheNeed::PagedRows;
      for (const Json& s : c.at("row_shape").items()) info.cache.row_shape.push_back(s.as_int());
      info.cache.rows_f32 = c.has("float32") && c.at("float32").as_bool();
      info.cache.window = (c.has("window") && !c.at("window").is_null()) ? (int)c.at("window").as_int() : 0;
    } else {
      info.cache.kind = CacheNeed::PagedKV;
      info.cache.kv_heads = (int)c.at("kv_heads").as_int();
      info.cache.head_dim = (int)c.at("head_dim").as_int();
      info.cache.window = c.has("window") ? (int)c.at("window").as_int() : 0;
    }
  }
  return info;
}

void foreign_call(uint64_t id, const char* op, StepContext* ctx, const Tensor* args, int n_args, const char* names,
                  Tensor* result) {
  if (!g_foreign.call) throw EngineError("a part implemented outside the library was called, but no call table is set");
  g_foreign_error.clear();
  if (ctx) ctx->ops.flush();        // whatever the part reads, it finds complete
  const int rc = g_foreign.call(id, op, ctx, args, n_args, names, result);
  if (rc != 0) throw EngineError(g_foreign_error.empty() ? std::string("a foreign part failed in '") + op + "'" : g_foreign_error);
}

// what all foreign parts share; Base is the family's interface
template <class Base> class Foreign : public Base {
 public:
  Foreign(uint64_t id, const std::string& prefix, const Json& description, const PartChildren& c)
      : Base(prefix), info(read_description(description)) {
    this->foreign_id = id;
    for (const auto& kv : c) {
      kids.push_back(kv.second);
      slots.push_back(kv.first);
    }
  }
  std::vector<std::string> child_slots() const override { return slots; }
  const char* kind_name() const override { return "foreign"; }
  std::vector<std::pair<std::string, TensorNeed>> tensors() const override { return info.tensors; }
  std::vector<std::shared_ptr<Part>> children() const override { return kids; }
  bool has_cache() const override { return info.has_cache; }
  CacheNeed cache_need() const override { return info.cache; }
  void load(WeightSource& src) override {
    std::vector<Tensor> ts;
    std::string names;
    for (const auto& kv : info.tensors) {
      if (!src.has(kv.first)) continue;
      ts.push_back(src.fetch(kv.first, kv.second));
      names += (names.empty() ? "" : "\n") + kv.first;
    }
    foreign_call(this->foreign_id, "load", nullptr, ts.data(), (int)ts.size(), names.c_str(), nullptr);
  }
  void prepare(Ops&, int max_seq) override {
    const std::string arg = std::to_string(max_seq);
    foreign_call(this->foreign_id, "prepare", nullptr, nullptr, 0, arg.c_str(), nullptr);
  }
  ForeignInfo info;
  std::vector<std::shared_ptr<Part>> kids;
  std::vector<std::string> slots;
};

class ForeignEmbedding final : public Foreign<EmbeddingPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Tensor& x) override { foreign_call(foreign_id, "forward", &ctx, &x, 1, "", nullptr); }
};
class ForeignNorm final : public Foreign<NormPart> {
 public:
  using Foreign::Foreign;
  Rows forward(StepContext& ctx, const Tensor& x, const int* rows, int64_t n_rows, bool) override {
    Tensor args[2] = {x, rows ? Tensor((void*)rows, DType::I32, {n_rows}) : Tensor()};
    Rows r;
    foreign_call(foreign_id, "forward", &ctx, args, 2, "", &r.t);
    return r;
  }
};
class ForeignPos final : public Foreign<PositionPart> {
 public:
  using Foreign::Foreign;
  void apply(StepContext& ctx, const Tensor& q, const Tensor& k) override {
    Tensor args[2] = {q, k};
    foreign_call(foreign_id, "apply", &ctx, args, 2, "", nullptr);
  }
};
class ForeignMixer final : public Foreign<MixerPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor args[2] = {h.materialize(ctx.ops), x};
    foreign_call(foreign_id, "forward", &ctx, args, 2, "", nullptr);
  }
};
class ForeignFFN final : public Foreign<FeedForwardPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Rows& h, const Tensor& x) override {
    Tensor args[2] = {h.materialize(ctx.ops), x};
    foreign_call(foreign_id, "forward", &ctx, args, 2, "", nullptr);
  }
};
class ForeignBlock final : public Foreign<BlockPart> {
 public:
  using Foreign::Foreign;
  void forward(StepContext& ctx, const Tensor& x) override { foreign_call(foreign_id, "forward", &ctx, &x, 1, "", nullptr); }
};
class ForeignHead final : public Foreign<HeadPart> {
 public:
  using Foreign::Foreign;
  Tensor forward(StepContext& ctx, const Rows& h) override {
    Tensor out;
    foreign_call(foreign_id, "forward", &ctx, &h.materialize(ctx.ops), 1, "", &out);
    return out;
  }
};
}  // namespace

void set_foreign_calls(const ForeignCalls& calls) { g_foreign = calls; }
void set_foreign_error(const std::string& message) { g_foreign_error = message; }
std::string take_foreign_error() {
  std::string m;
  m.swap(g_foreign_error);
  return m;
}

std::shared_ptr<Part> make_foreign_part(const std::string& family, uint64_t id, const std::string& prefix,
                                        const Json& description, const PartChildren& children) {
  if (family == "embedding") return std::make_shared<ForeignEmbedding>(id, prefix, description, children);
  if (family == "norm") return std::make_shared<ForeignNorm>(id, prefix, description, children);
  if (family == "pos") return std::make_shared<ForeignPos>(id, prefix, description, children);
  if (family == "mixer") return std::make_shared<ForeignMixer>(id, prefix, description, children);
  if (family == "ffn") return std::make_shared<ForeignFFN>(id, prefix, description, children);
  if (family == "block") return std::make_shared<ForeignBlock>(id, prefix, description, children);
  if (family == "head") return std::make_shared<ForeignHead>(id, prefix, description, children);
  if (family == "filter") throw ConfigError("a filter part is implemented in the library or in a plugin loaded into it, not through the call table");
  throw ConfigError("unknown part family '" + family + "'");
}

}  // namespace tinyinfer

// small HIP helpers the rotary part needs (kept out of the class so that this file's other code
// does not depend on the HIP headers)
#include <hip/hip_runtime_api.h>
namespace tinyinfer {
namespace {
void RotaryNeox::upload(void* dst, const void* src, size_t bytes) {
  if (hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice) != hipSuccess) throw KernelError("rotary: copying the inverse frequencies failed");
}
void Sinusoidal::upload(void* dst, const void* src, size_t bytes) {
  if (hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice) != hipSuccess) throw KernelError("sinusoidal positions: copying the frequencies failed");
}
float DiffAttention::lambda_of(const Tensor l[4], int dk, double diff, bool on_host) {
  std::vector<float> host((size_t)4 * dk);
  for (int i = 0; i < 4; ++i) {
    if (on_host) {
      memcpy(host.data() + (size_t)i * dk, l[i].data, (size_t)dk * 4);
    } else if (hipDeviceSynchronize() != hipSuccess ||
               hipMemcpy(host.data() + (size_t)i * dk, l[i].data, (size_t)dk * 4, hipMemcpyDeviceToHost) != hipSuccess) {
      throw KernelError("diff_attention: reading the lambda vectors back failed");
    }
  }
  float s1 = 0.f, s2 = 0.f;
  for (int d = 0; d < dk; ++d) {
    s1 = std::fmaf(host[d], host[(size_t)dk + d], s1);
    s2 = std::fmaf(host[(size_t)2 * dk + d], host[(size_t)3 * dk + d], s2);
  }
  return std::exp(s1) - std::exp(s2) + (float)diff;
}
void DecayAttention::put_floats(const Tensor& dst, const std::vector<float>& values, bool on_host) {
  if (on_host) {
    memcpy(dst.data, values.data(), values.size() * 4);
    return;
  }
  if (hipMemcpy(dst.data, values.data(), values.size() * 4, hipMemcpyHostToDevice) != hipSuccess)
    throw KernelError("copying a part's constants to the device failed");
}
void RMSNorm::plus_one(const Tensor& w, const Tensor& out, bool on_host) {
  const size_t n = (size_t)w.numel();
  if (on_host) {
    for (size_t i = 0; i < n; ++i) out.ptr<float>()[i] = 1.0f + w.ptr<float>()[i];
    return;
  }
  std::vector<float> host(n);
  // the weight may still be on its way from the file: wait for every stream before reading it back
  if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(host.data(), w.data, n * 4, hipMemcpyDeviceToHost) != hipSuccess)
    throw KernelError("rmsnorm: reading the weight back failed");
  for (float& v : host) v = 1.0f + v;
  if (hipMemcpy(out.data, host.data(), n * 4, hipMemcpyHostToDevice) != hipSuccess) throw KernelError("rmsnorm: writing the gain failed");
}
void RMSNorm::spread(const Tensor& one, const Tensor& all, bool on_host) {
  float g = 0.f;
  if (on_host) {
    g = *one.ptr<float>();
    for (int64_t i = 0; i < all.numel(); ++i) all.ptr<float>()[i] = g;
    return;
  }
  // the number may still be on its way from the file: wait for every stream before reading it back
  if (hipDeviceSynchronize() != hipSuccess || hipMemcpy(&g, one.data, 4, hipMemcpyDeviceToHost) != hipSuccess)
    throw KernelError("rmsnorm: reading the scalar gain back failed");
  std::vector<float> host((size_t)all.numel(), g);
  if (hipMemcpy(all.data, host.data(), host.size() * 4, hipMemcpyHostToDevice) != hipSuccess)
    throw KernelError("rmsnorm: spreading the scalar gain failed");
}
}  // namespace
}  // namespace tinyinfer
