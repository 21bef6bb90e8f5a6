"""Dubozen without a GPU: the configuration reader, the model as data (tensors, run order, cache needs), and the plain
implementation's mechanisms against other ways of writing the same formulas."""
import copy
import math

import numpy as np
import pytest

import dubozen_models as dm
from plain import dubozen_plain as plain


def spec_of(config):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import config_and_spec
    return config_and_spec(config)


def test_architecture_is_registered():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import registered_architectures
    assert "Dubozen" in registered_architectures()


@pytest.mark.parametrize("name", sorted(dm.CONFIGS))
def test_spec_asks_for_the_tensors_of_the_configuration(name):
    from tinyinfer_amd.models.model import Model
    config = dm.CONFIGS[name]
    typed, spec = spec_of(config)
    model = Model(spec)
    want = {k: tuple(v.shape) for k, v in dm.draw_weights(config, 1).items()}
    got = {k: tuple(v.shape) for k, v in model.tensors().items() if not v.optional}
    assert got == want
    assert typed["width"] == config["width"] and typed["vocab"] == config["vocab"]


def test_streams_are_opened_and_closed_by_layers_of_their_own():
    from tinyinfer_amd.models.model import Model
    _, spec = spec_of(dm.CONFIGS["streams"])
    # five real layers, then the block that opens the streams (5) and the one that sums them (6)
    assert spec.run_order() == [5, 0, 1, 2, 3, 4, 6]
    model = Model(spec)
    kv = sorted((n.kv_heads, n.head_dim, n.v_dim, c) for n, c in model.cache_groups if type(n).__name__ == "PagedKVNeed")
    # keys and values per softmax attention: (kv heads, key size, value size if it differs) and how many layers share the need
    assert kv == [(1, 8, 10, 1), (1, 16, None, 1), (2, 8, None, 1), (2, 12, 24, 1), (2, 16, 24, 1)]
    # values smaller than keys of a size the matrix cores take are padded to the keys' size in the pages: no value size of their own
    kv = sorted((n.kv_heads, n.head_dim, n.v_dim) for n, c in Model(spec_of(dm.CONFIGS["squares"])[1]).cache_groups if type(n).__name__ == "PagedKVNeed")
    assert (1, 32, None) in kv and not any(v == 16 for _, _, v in kv)
    states = sorted((tuple(n.shape), c) for n, c in model.cache_groups if type(n).__name__ == "StateNeed")
    # the linear attention's memory per request: heads x (keys x values)
    assert states == [((2, 96), 1), ((3, 96), 1)]
    _, spec = spec_of(dm.CONFIGS["plain"])
    assert spec.run_order() == [0, 1, 2, 3]      # one residual: no streams to open


def test_defaults_are_filled_in():
    config = copy.deepcopy(dm.CONFIGS["plain"])
    m = config["layers"][1]["mixer"]
    del m["kv_heads"], m["vdim"], m["scale"], m["v_mix"]
    del config["layers"][0]["mixer"]["left_scale"]
    del config["layers"][2]["mlp"]["router"]["scale"]
    typed, _ = spec_of(config)
    got = typed["layers"][1]["mixer"]
    assert got["kv_heads"] == 5 and got["vdim"] == 10 and got["v_mix"] is False and abs(got["scale"] - 10 ** -0.5) < 1e-12
    assert typed["layers"][0]["mixer"]["left_scale"] == 1.0
    assert typed["layers"][2]["mlp"]["router"]["scale"] == 1.0
    assert typed["streams"] is None and typed["layers"][1]["mlp"] is None


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0]["mixer"].update(heads=5), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "dims"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=20), "kv_heads' and 'vdim"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(vdim=12), "vdim"),
    (lambda c: c["layers"][1]["mixer"]["right"].update(decay=[0.5, 0.6]), "decay"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=1, count=6), "groups"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][1].update(type="mamba"), "mamba"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "sparse"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c.update(streams=17), "streams"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0]["mixer"].pop("dim"), "dim"),
])
def test_what_is_not_served_is_refused_by_name(change, word):
    from tinyinfer_amd import ConfigError
    config = copy.deepcopy(dm.CONFIGS["streams"])
    change(config)
    with pytest.raises(ConfigError) as e:
        spec_of(config)
    assert word in str(e.value)


# ------------------------------------------------------------------------ the plain implementation against itself
def test_layer_norm_takes_mean_and_variance():
    rng = np.random.default_rng(0)
    x = rng.normal(3.0, 2.0, size=(5, 33))
    g = rng.normal(1.0, 0.2, size=33)
    y = plain.layer_norm(x, g, 0.0) / g
    assert np.abs(y.mean(axis=-1)).max() < 1e-12 and np.abs(y.var(axis=-1) - 1.0).max() < 1e-12
    # an RMS norm of the same rows is something else: the mean stays
    assert np.abs(plain.rms_norm(x, g, 0.0) / g - y).max() > 0.5


def test_a_sink_is_a_key_with_no_value():
    """exp(sink) in the denominator = one more key with score `sink` (not scaled) whose value is zero."""
    rng = np.random.default_rng(1)
    T = 9
    s = rng.normal(size=(T, T)) * 2
    sink = 0.7
    p = plain.causal_softmax(s, sink)
    wide = np.concatenate([s, np.full((T, 1), sink)], axis=1)
    vis = np.concatenate([np.tril(np.ones((T, T), dtype=bool)), np.ones((T, 1), dtype=bool)], axis=1)
    e = np.where(vis, np.exp(wide - wide.max()), 0.0)
    ref = e / e.sum(axis=1, keepdims=True)
    assert np.abs(p - ref[:, :T]).max() < 1e-12
    assert (p.sum(axis=1) < 1.0).all() and np.abs(plain.causal_softmax(s).sum(axis=1) - 1.0).max() < 1e-12


def test_linear_attention_is_a_decayed_sum_over_the_past():
    """o_t = sum_(j <= t) decay^(t - j) (q_t . k_j) v_j: the recurrence unrolled."""
    rng = np.random.default_rng(2)
    W, T = 12, 17
    m = dict(heads=2, dim=3, vdim=5, decay=[0.9, 0.5])
    w = {"r.q": rng.normal(size=(6, W)), "r.k": rng.normal(size=(6, W)), "r.v": rng.normal(size=(10, W)), "r.g": rng.normal(size=(10, W)),
         "r.o": np.eye(10), "r.norm": np.ones(10)}
    h = rng.normal(size=(T, W))
    got = plain.decayed_linear_attention(h, m, w, "r", 1e-6)
    q = plain.silu(h @ w["r.q"].T).reshape(T, 2, 3)
    k = plain.silu(h @ w["r.k"].T).reshape(T, 2, 3)
    v = plain.silu(h @ w["r.v"].T).reshape(T, 2, 5)
    o = np.zeros((T, 2, 5))
    for j in range(2):
        for t in range(T):
            for u in range(t + 1):
                o[t, j] += m["decay"][j] ** (t - u) * (q[t, j] @ k[u, j]) * v[u, j]
    want = plain.rms_norm(o.reshape(T, 10), np.ones(10), 1e-6) * plain.sigmoid(h @ w["r.g"].T)
    assert np.abs(got - want).max() < 1e-10


def test_router_keeps_the_best_groups_and_weighs_without_the_correction():
    rng = np.random.default_rng(3)
    W, E = 8, 6
    w = {"m.router": rng.normal(size=(E, W)), "m.correction": np.array([-3.0, -3.0, 0.1, 0.0, -0.2, 0.3])}
    h = rng.normal(size=(40, W))
    r = dict(experts=E, top=2, scale=1.5, groups=dict(count=3, keep=1))
    ids, wts = plain.route(h, r, w, "m")
    s = plain.sigmoid(h @ w["m.router"].T)
    for t in range(40):
        assert ids[t, 0] // 2 == ids[t, 1] // 2                      # both from one group of two neighbours
        assert ids[t, 0] // 2 != 0                                    # the group whose corrections are far below never wins
        assert abs(wts[t].sum() - 1.5) < 1e-9                         # renormalised, then scaled
        assert abs(wts[t, 0] / wts[t, 1] - s[t, ids[t, 0]] / s[t, ids[t, 1]]) < 1e-9      # ratios of the uncorrected scores
    # all groups kept and no correction: the plain top-2 of the scores
    w["m.correction"] = np.zeros(E)
    ids, _ = plain.route(h, dict(experts=E, top=2, scale=1.0, groups=dict(count=3, keep=3)), w, "m")
    assert (np.sort(ids, axis=1) == np.sort(np.argsort(-s, axis=1)[:, :2], axis=1)).all()
    # negative choice scores everywhere: experts outside the kept groups still cannot be chosen
    w["m.correction"] = np.full(E, -5.0) + np.array([0, 0, 0, 0, 1.0, 1.0])
    ids, _ = plain.route(h, r, w, "m")
    assert (ids // 2 == 2).all()


def test_streams_of_equal_weights_are_a_plain_residual():
    """With one stream and in = mix = out = 1 a layer on streams is x + y."""
    config = copy.deepcopy(dm.CONFIGS["single"])
    w = dm.as_float64(dm.draw_weights(config, 4))
    for k in w:
        if ".hc" in k:
            w[k] = np.ones_like(w[k])
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    a = plain.forward(config, w, toks)
    del config["streams"]
    b = plain.forward(config, {k: v for k, v in w.items() if ".hc" not in k}, toks)
    assert np.abs(a - b).max() < 1e-10


def test_every_learned_tensor_moves_the_logits():
    config = dm.CONFIGS["streams"]
    w = dm.as_float64(dm.draw_weights(config, 5))
    toks = [int(t) for t in np.random.default_rng(6).integers(0, config["vocab"], size=24)]
    base = plain.forward(config, w, toks)
    unused = {"l0.mix.vmix"}      # the first layer that mixes values has nothing to mix them with
    for name in w:
        if name.startswith(("l1.mlp.e", "l4.mlp.")):
            continue                # an expert that no token of this prompt chose moves nothing; one expert of four, its weight
                                    # renormalised, hears of its router only when the choice changes
        changed = dict(w)
        changed[name] = w[name] * 1.3 + 0.05
        moved = np.abs(plain.forward(config, changed, toks) - base).max()
        assert (moved < 1e-12) == (name in unused), (name, moved)


def test_values_of_the_first_mixing_layer_reach_the_later_ones():
    config = dm.CONFIGS["streams"]
    w = dm.as_float64(dm.draw_weights(config, 7))
    toks = [int(t) for t in np.random.default_rng(8).integers(0, config["vocab"], size=12)]
    base = plain.forward(config, w, toks)
    off = dict(w)
    off["l2.mix.vmix"] = np.zeros(())
    assert np.abs(plain.forward(config, off, toks) - base).max() > 1e-3
    # with lambda = 1 layer 2 attends over layer 0's values alone: its own value projection no longer matters
    one = dict(w)
    one["l2.mix.vmix"] = np.ones(())
    a = plain.forward(config, one, toks)
    one["l2.mix.v"] = w["l2.mix.v"] * 0.0
    assert np.abs(plain.forward(config, one, toks) - a).max() < 1e-10


def test_gelu_is_the_tanh_form():
    z = np.linspace(-4, 4, 33)
    exact = 0.5 * z * (1.0 + np.array([math.erf(v / math.sqrt(2.0)) for v in z]))
    assert np.abs(plain.gelu_tanh(z) - exact).max() < 5e-3 and np.abs(plain.gelu_tanh(z) - exact).max() > 1e-5
