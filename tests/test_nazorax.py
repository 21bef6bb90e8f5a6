"""Nazorax without a GPU: the configuration reader, the model as data (tensors, run order, cache needs), and the plain
implementation's mechanisms against other ways of writing the same formulas."""
import copy
import math

import numpy as np
import pytest

import nazorax_models as nm
from plain import nazorax_plain as plain


def spec_of(config):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import config_and_spec
    return config_and_spec(config)


def test_architecture_is_registered():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.registry import registered_architectures
    assert "Nazorax" in registered_architectures()


@pytest.mark.parametrize("name", sorted(nm.CONFIGS))
def test_spec_asks_for_the_tensors_of_the_configuration(name):
    from tinyinfer_amd.models.model import Model
    config = nm.CONFIGS[name]
    typed, spec = spec_of(config)
    model = Model(spec)
    want = {k: tuple(v.shape) for k, v in nm.draw_weights(config, 1).items()}
    got = {k: tuple(v.shape) for k, v in model.tensors().items() if not v.optional}
    assert got == want
    assert typed["width"] == config["width"] and typed["vocab"] == config["vocab"]


def test_run_order_and_caches_of_a_loop():
    from tinyinfer_amd.models.model import Model
    config = nm.CONFIGS["looped"]
    _, spec = spec_of(config)
    # four real layers, then the block that keeps the embedding's output (4) and the one that mixes it in (5): kept right
    # behind the embedding, mixed in before each of the three passes over layers 1 and 2
    assert spec.run_order() == [4, 0, 5, 1, 2, 5, 1, 2, 5, 1, 2, 3]
    model = Model(spec)
    kv = sorted((n.kv_heads, n.head_dim, n.v_dim, n.window, c) for n, c in model.cache_groups if type(n).__name__ == "PagedKVNeed")
    # a cache layer per run: layer 2 runs three times, layer 0 once
    assert kv == [(1, 16, 24, 21, 1), (2, 8, None, 40, 3)]
    rows = sorted((tuple(n.row_shape), c) for n, c in model.cache_groups if type(n).__name__ == "PagedRowsNeed")
    # the latent layers keep kv_rank + rot_dim numbers a token: layer 1 three times, layer 3 once
    assert rows == [((24,), 1), ((32,), 3)]
    assert plain.run_order(config) == [(0, False), (1, True), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]


def test_a_loop_from_the_first_layer_and_no_loop():
    _, spec = spec_of(nm.CONFIGS["odd"])
    assert spec.run_order() == [3, 4, 0, 1, 2]
    assert plain.run_order(nm.CONFIGS["odd"]) == [(0, True), (1, False), (2, False)]
    _, spec = spec_of(nm.CONFIGS["wide"])
    assert spec.run_order() == [0, 1, 2]
    from tinyinfer_amd.models.model import Model
    assert "loop.in" not in Model(spec).tensors()


def test_pages_of_a_latent_layer_hold_the_latents_twice_where_the_matrix_cores_serve_the_sizes():
    """kv_rank + rot_dim numbers a token, and kv_rank more (the latents transposed) where the latent is a multiple of 16, latent and
    key part together a multiple of 8, the unrotated query size a multiple of 8 and the value size a multiple of 16."""
    from tinyinfer_amd.models.model import Model
    _, spec = spec_of(nm.CONFIGS["wide"])
    rows = [tuple(n.row_shape) for n, _ in Model(spec).cache_groups if type(n).__name__ == "PagedRowsNeed"]
    assert rows == [(64 + 16 + 64,)]
    config = copy.deepcopy(nm.CONFIGS["wide"])
    config["layers"][1]["mixer"]["vdim"] = 40                # values that are no multiple of 16: rows only
    _, spec = spec_of(config)
    rows = [tuple(n.row_shape) for n, _ in Model(spec).cache_groups if type(n).__name__ == "PagedRowsNeed"]
    assert rows == [(64 + 16,)]


@pytest.mark.parametrize("change,word", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].__setitem__("type", "mlstm"), "mlstm"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 2), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7), "dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), "dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 10), "dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("kv_rank", 900), "768"),
    (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "size"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "sparse"), "sparse"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 6), "top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "limit"),
    (lambda c: c["layers"][1]["mlp"]["shared"].pop("ff"), "ff"),
    (lambda c: c["loop"].__setitem__("stop", 9), "stop"),
    (lambda c: c["loop"].__setitem__("times", 0), "times"),
])
def test_bad_configurations_are_refused_by_name(change, word):
    from tinyinfer_amd.config.base import ConfigError
    from tinyinfer_amd.models.model import Model
    config = copy.deepcopy(nm.CONFIGS["looped"])
    change(config)
    with pytest.raises((ConfigError, ValueError)) as e:
        _, spec = spec_of(config)
        Model(spec)
    assert word in str(e.value)


def test_defaults_are_filled_in():
    config = copy.deepcopy(nm.CONFIGS["looped"])
    a = config["layers"][2]["mixer"]
    for key in ("kv_heads", "vdim", "scale", "mask", "rot"):
        a.pop(key)
    config["layers"][1]["mlp"].pop("shared")
    config.pop("loop")
    typed, spec = spec_of(config)
    t = typed["layers"][2]["mixer"]
    assert t["kv_heads"] == 4 and t["vdim"] == 8 and t["mask"] is None and t["rot"] is None and abs(t["scale"] - 8 ** -0.5) < 1e-12
    assert typed["loop"] is None and typed["layers"][1]["mlp"]["shared"] is None
    from tinyinfer_amd.models.model import Model
    names = Model(spec).tensors()
    assert not any("shared" in n for n in names) and "loop.in" not in names and spec.run_order() == [0, 1, 2, 3]


# ------------------------------------------------------------------------------ the plain implementation
def test_dynamic_tanh_is_neither_a_mean_nor_a_variance():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(3, 10))
    w = {"n": rng.normal(size=10), "n.b": rng.normal(size=10), "n.alpha": np.asarray(0.7)}
    y = plain.dynamic_tanh(x, w, "n")
    for i in range(3):
        for c in range(10):
            assert abs(y[i, c] - (math.tanh(0.7 * x[i, c]) * w["n"][c] + w["n.b"][c])) < 1e-12
    # every entry depends on its own input alone
    x2 = x.copy()
    x2[0, 3] += 5.0
    y2 = plain.dynamic_tanh(x2, w, "n")
    assert np.array_equal(np.delete(y2, 3, axis=1), np.delete(y, 3, axis=1))


def test_window_and_causal_masks():
    vis = plain.window_mask(9, 3)
    for i in range(9):
        assert [j for j in range(9) if vis[i, j]] == [j for j in range(9) if 0 <= i - j < 3]
    vis = plain.window_mask(5, None)
    assert np.array_equal(vis, np.tril(np.ones((5, 5), dtype=bool)))


def test_a_sink_is_a_key_without_a_value():
    rng = np.random.default_rng(1)
    s = rng.normal(size=(4, 4)) * 2
    vis = plain.window_mask(4, None)
    v = rng.normal(size=(4, 3))
    sink = 0.8
    got = plain.softmax_rows(s, vis, sink) @ v
    # the same with a fifth key whose score is the sink and whose value is zero
    s5 = np.concatenate([s, np.full((4, 1), sink)], axis=1)
    vis5 = np.concatenate([vis, np.ones((4, 1), dtype=bool)], axis=1)
    want = plain.softmax_rows(s5, vis5) @ np.concatenate([v, np.zeros((1, 3))])
    assert np.abs(got - want).max() < 1e-12
    assert (plain.softmax_rows(s, vis, sink).sum(axis=1) < 1.0).all()


def test_rotation_turns_pairs_half_a_head_apart_and_yarn_slows_the_slow_ones():
    rot = dict(base=100.0, dims=6)
    x = np.arange(1.0, 11.0).reshape(1, 10)
    y = plain.rotate_half(np.repeat(x, 4, axis=0), range(4), rot)
    assert np.array_equal(y[:, 6:], np.repeat(x, 4, axis=0)[:, 6:])      # the rest of the head passes
    assert np.array_equal(y[0], x[0])                                    # position 0 turns nothing
    for i in range(3):
        a = 3 * 100.0 ** (-2.0 * i / 6)
        assert abs(y[3, i] - (x[0, i] * math.cos(a) - x[0, i + 3] * math.sin(a))) < 1e-12
        assert abs(y[3, i + 3] - (x[0, i + 3] * math.cos(a) + x[0, i] * math.sin(a))) < 1e-12
    f_plain, mag_plain = plain.frequencies(dict(base=10000.0, dims=16))
    f, mag = plain.frequencies(dict(base=10000.0, dims=16, scaling=nm.yarn(4.0, 64, 8.0, 1.0)))
    assert mag_plain == 1.0 and abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    assert abs(f[0] - f_plain[0]) < 1e-15 and abs(f[-1] - f_plain[-1] / 4.0) < 1e-15      # fast ones stay, slow ones are divided
    assert all(f_plain[i] / 4.0 - 1e-15 <= f[i] <= f_plain[i] + 1e-15 for i in range(8))


def test_latent_attention_equals_attention_over_the_latents_themselves():
    """Keys and values per head from the latent, against the form that attends over the latents with the query taken through
    W_uk and maps the weighted latent through W_uv afterwards."""
    config = nm.CONFIGS["looped"]
    m = config["layers"][1]["mixer"]
    w = nm.as_float64(nm.draw_weights(config, 4))
    rng = np.random.default_rng(2)
    T = 13
    h = rng.normal(size=(T, config["width"]))
    pre = "l1.mix"
    got = plain.latent_attention(h, w, pre, m, 1e-5)
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[pre + ".q"].T).reshape(T, H, d + r)
    down = h @ w[pre + ".dkv"].T
    c = plain.rms_unit(down[:, :R], 1e-5) * w[pre + ".dkv.norm"]
    kr = plain.rotate_half(down[:, R:], range(T), m["rot"])
    out = np.zeros((T, H, dv))
    for hd in range(H):
        uk, uv = w[pre + ".uk"][hd * d:(hd + 1) * d], w[pre + ".uv"][hd * dv:(hd + 1) * dv]
        for i in range(T):
            qa = q[i, hd, :d] @ uk                                        # [R]
            qr = plain.rotate_half(q[i:i + 1, hd, d:], [i], m["rot"])[0]
            s = np.array([(qa @ c[j] + qr @ kr[j]) * m["scale"] for j in range(i + 1)])
            top = max(s.max(), w[pre + ".sink"][hd])
            p = np.exp(s - top)
            p = p / (p.sum() + math.exp(w[pre + ".sink"][hd] - top))
            out[i, hd] = uv @ (p @ c[:i + 1])
    want = out.reshape(T, H * dv) @ w[pre + ".o"].T
    assert np.abs(got - want).max() < 1e-10


def test_router_weights_are_a_softmax_over_the_chosen_logits():
    rng = np.random.default_rng(3)
    h, wr = rng.normal(size=(6, 8)), rng.normal(size=(5, 8))
    idx, wt = plain.router_choice(h, wr, 3)
    z = h @ wr.T
    for t in range(6):
        order = sorted(range(5), key=lambda e: (-z[t, e], e))[:3]
        assert list(idx[t]) == order
        e = np.exp(z[t, order])
        assert np.abs(wt[t] - e / e.sum()).max() < 1e-12
    # equal logits: the lower index first
    idx, wt = plain.router_choice(np.ones((1, 2)), np.ones((4, 2)), 2)
    assert list(idx[0]) == [0, 1] and np.allclose(wt, 0.5)


def test_clamped_expert_clamps_gate_from_above_and_up_on_both_sides():
    w = {"e.gate": np.array([[1.0], [1.0], [1.0]]), "e.up": np.array([[1.0], [-1.0], [0.1]]), "e.down": np.eye(3)}
    y = plain.clamped_expert(np.array([[5.0]]), w, "e", 2.0)[0]
    g = 2.0
    act = g / (1.0 + math.exp(-1.702 * g))
    assert abs(y[0] - act * 3.0) < 1e-12 and abs(y[1] - act * -1.0) < 1e-12 and abs(y[2] - act * 1.5) < 1e-12
    # a strongly negative gate is not clamped
    y = plain.clamped_expert(np.array([[-5.0]]), w, "e", 2.0)[0]
    assert abs(y[2] - (-5.0 / (1.0 + math.exp(1.702 * 5.0))) * 0.5) < 1e-12


def test_every_learned_piece_changes_the_logits():
    """A tensor that is forgotten or put in the wrong place shows: zeroing or shifting any one of them moves the logits."""
    config = nm.CONFIGS["looped"]
    w = nm.as_float64(nm.draw_weights(config, 7))
    toks = list(np.random.default_rng(5).integers(0, config["vocab"], size=30))
    base = plain.forward(config, w, toks)
    for name in ("loop.in", "l0.mix.k.b", "l0.mlp.down.b", "l1.mix.sink", "l1.mix.dkv.norm", "l1.mlp.shared.up", "l1.norm1.alpha",
                 "l2.norm1.b", "l3.mix.uk", "final.norm.b"):
        w2 = dict(w)
        w2[name] = w[name] * 0.5 + 0.3
        assert np.abs(plain.forward(config, w2, toks) - base).max() > 1e-3, name
    # the window: a token far behind it does not reach the last position through layer 0 alone, but one inside does
    only = dict(config, layers=config["layers"][:1], loop=None)
    a = plain.forward(only, w, toks)
    far, near = list(toks), list(toks)
    far[3] = (far[3] + 1) % config["vocab"]
    near[29 - 20] = (near[29 - 20] + 1) % config["vocab"]                 # distance 20 < 21
    assert np.abs(plain.forward(only, w, far)[-1] - a[-1]).max() == 0.0
    assert np.abs(plain.forward(only, w, near)[-1] - a[-1]).max() > 1e-6
    edge = list(toks)
    edge[29 - 21] = (edge[29 - 21] + 1) % config["vocab"]                 # distance 21: just outside
    assert np.abs(plain.forward(only, w, edge)[-1] - a[-1]).max() == 0.0
