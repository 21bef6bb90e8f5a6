"""Dubozen on the GPU against the plain implementation: every mechanism alone through the kernels' own object, and the
engine under every way of cutting the work (each request whole; most of it in one step and its last tokens one by
one; portions of changing size down to two tokens; up to four live requests mixed, with so few pages and slots that they
are used again), in 32-bit and in bfloat16, and greedy generation through the entry point and the scheduler."""
import math

import numpy as np
import pytest
import torch

import dubozen_models as dm
import traces
from helpers import random_tokens
from plain import dubozen_plain as plain

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# rms of (engine - plain) over rms of the plain logits, per position.  float32: rounding of 32-bit sums against float64.
# bfloat16: operands of every product, cached keys and values and the queries are rounded to 8 bits, which moves the logits
# by a per cent or two, while a lost key, a forgotten sink, a lost state or a wrong expert moves them by tens of per cent.
# Where two experts' choice scores lie within that rounding of each other, bfloat16 may pick the other one with nothing
# wrong: in bfloat16 the bound holds for all but 8 % of the positions and the median error stays under 2 %.
TOL = {"float32": 2e-4, "bfloat16": 8e-2}


@pytest.fixture(scope="module")
def ops():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.ops.kernels import get_ops
    return get_ops()


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a)).to(dtype).to("cuda")


def f64(t):
    return t.detach().to("cpu", torch.float64).numpy()


def bf16_round(a):
    return torch.as_tensor(np.asarray(a, dtype=np.float32)).to(torch.bfloat16).to(torch.float64).numpy()


def f32_round(a):
    return np.asarray(a, dtype=np.float32).astype(np.float64)


def paged(rng, n_tokens, P, extra_pages=3):
    n_pages = -(-n_tokens // P)
    ids = rng.permutation(n_pages + extra_pages)[:n_pages]
    return np.asarray(ids, dtype=np.int32)[None, :], n_pages + extra_pages


# ---------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("W", [50, 192, 1030])
def test_layer_norm(ops, dtype, W):
    rng = np.random.default_rng(W)
    x = rng.normal(1.5, 3.0, size=(37, W))          # a mean far from zero: an RMS norm in its place would show
    g = rng.normal(1.0, 0.3, size=W)
    want = plain.layer_norm(f32_round(x), f32_round(g), 1e-5)
    tol = 3e-5 if dtype == "float32" else 2.0 ** -7
    out = torch.empty(37, W, device="cuda", dtype=DT[dtype])
    ops.layernorm(dev(x), dev(g), 1e-5, out)
    assert np.abs(f64(out) - want).max() < tol * np.abs(want).max()
    rows = np.array([36, 0, 5, 5, 17], dtype=np.int32)
    some = torch.empty(len(rows), W, device="cuda", dtype=DT[dtype])
    ops.layernorm(dev(x), dev(g), 1e-5, some, dev(rows, torch.int32))
    assert np.array_equal(f64(some), f64(out)[rows])
    if dtype == "float32":                          # in place on 32-bit rows: what the embedding's norm does
        xs = dev(x)
        ops.layernorm(xs, dev(g), 1e-5, xs)
        assert np.array_equal(f64(xs), f64(out))


@pytest.mark.parametrize("S", [1, 2, 3, 5, 16])
def test_streams_read_and_written(ops, S):
    """A sublayer's input is the norm of a weighted sum of the streams; its output goes back into all of them at once
    beside a mixing of the old ones (the new stream t must not see the new stream t - 1)."""
    rng = np.random.default_rng(S)
    M, W = 19, 70
    xs = rng.normal(size=(S, M, W))
    coef, back = rng.normal(0.5, 0.5, size=S), rng.normal(1.0, 0.5, size=S)
    mix = np.eye(S) + rng.normal(0.0, 0.4, size=(S, S))
    g = rng.normal(1.0, 0.2, size=W)
    y = rng.normal(size=(M, W))
    x32, c32, b32, m32, y32 = f32_round(xs), f32_round(coef), f32_round(back), f32_round(mix), f32_round(y)
    u = np.einsum("s,smw->mw", c32, x32)
    streams = dev(xs)
    for dtype in ("float32", "bfloat16"):
        out = torch.empty(M, W, device="cuda", dtype=DT[dtype])
        ops.layernorm_mixed(streams, dev(coef), dev(g), 1e-6, out)
        want = plain.layer_norm(u, f32_round(g), 1e-6)
        assert np.abs(f64(out) - want).max() < (5e-5 if dtype == "float32" else 2.0 ** -7) * np.abs(want).max()
    got_u = torch.empty(M, W, device="cuda")
    ops.hyper_combine(streams, dev(coef), got_u)
    assert np.abs(f64(got_u) - u).max() < 1e-5
    ops.hyper_combine(streams, None, got_u)
    assert np.abs(f64(got_u) - x32.sum(axis=0)).max() < 1e-5
    ops.hyper_write(streams, dev(mix), dev(back), dev(y))
    want = np.einsum("st,smw->tmw", m32, x32) + b32[:, None, None] * y32[None]
    assert np.abs(f64(streams) - want).max() < 1e-5 * max(1.0, np.abs(want).max())
    # two branches left apart and the next sublayer's read in the same pass: the same bits as the kernels one after the other
    y2 = rng.normal(size=(M, W))
    a, b = dev(xs), dev(xs)
    both = torch.empty(M, W, device="cuda")
    ops.scaled_add(both.zero_(), dev(y), torch.full((W,), 0.6, device="cuda"), dev(y2), torch.full((W,), 0.5, device="cuda"))
    want2 = np.einsum("st,smw->tmw", m32, x32) + b32[:, None, None] * (0.6 * y32 + 0.5 * f32_round(y2))[None]
    for dtype in ("float32", "bfloat16"):
        a.copy_(dev(xs))
        b.copy_(dev(xs))
        out1 = torch.empty(M, W, device="cuda", dtype=DT[dtype])
        out2 = torch.empty(M, W, device="cuda", dtype=DT[dtype])
        ops.hyper_write(a, dev(mix), dev(back), dev(y), dev(y2), 0.6, 0.5)
        ops.layernorm_mixed(a, dev(coef), dev(g), 1e-6, out1)
        ops.hyper_write(b, dev(mix), dev(back), dev(y), dev(y2), 0.6, 0.5, dev(coef), dev(g), 1e-6, out2)
        assert np.abs(f64(a) - want2).max() < 1e-5 * max(1.0, np.abs(want2).max())
        assert np.array_equal(f64(a), f64(b)) and np.array_equal(f64(out1), f64(out2))
    x0 = dev(y)
    ops.hyper_spread(x0, streams)
    assert all(np.array_equal(f64(streams[s]), f64(x0)) for s in range(S))


def rotation_inputs(rot, n_table):
    if not rot or not rot["dims"]:
        return None, None
    half = rot["dims"] // 2
    f = np.array([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(half)])
    ang = np.arange(n_table)[:, None] * f[None, :]
    return dev(f), dev(np.stack([np.cos(ang), np.sin(ang)], axis=-1))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv,dk,dv,P,rot_dims,normed,from_keys,gate,sink", [
    (4, 2, 16, 24, 16, 8, False, False, 1, True), (3, 3, 7, 7, 4, 6, True, True, 2, False), (6, 1, 40, 33, 64, 40, True, False, 1, True),
    (2, 2, 64, 64, 16, 32, True, True, 2, True), (2, 1, 64, 32, 16, 0, False, False, 0, True), (3, 1, 24, 16, 8, 12, False, False, 2, False),
    (8, 2, 128, 128, 32, 64, True, True, 0, False), (1, 1, 256, 256, 16, 2, False, False, 1, True)])
def test_gated_attention(ops, dtype, heads, kv, dk, dv, P, rot_dims, normed, from_keys, gate, sink):
    """The projections of a whole request get their per-head norms and the rotation of their first entries and go into the
    pages in three portions (the last a single token); then the attention of every row with its sink and its gate.  The last
    row's query points at key 1, far back among hundreds, and key 0 is as strong a second time: losing either shows; the first
    rows see one, two, three keys, where the sink weighs most."""
    rng = np.random.default_rng(dk * 1000 + dv + heads)
    T = 333
    scale = 1.3 / math.sqrt(dk)
    per = heads // kv
    nq, nk, nv = heads * dk, kv * dk, 0 if from_keys else kv * dv
    ng = heads * dv if gate == 1 else heads if gate == 2 else 0
    pad = 3                                                   # columns of another part of the stacked projection in between
    proj = rng.normal(size=(T, nq + nk + nv + pad + ng))
    q_w = rng.normal(1.0, 0.3, size=dk) if normed else None
    k_w = rng.normal(1.0, 0.3, size=dk) if normed else None
    # a far key made to stand out: on the entries that are not rotated (all of them where nothing is) key 1 and query T - 1 agree
    free = slice(rot_dims, dk) if rot_dims < dk else None
    if free is not None:
        for h in range(kv):
            proj[1, nq + h * dk:nq + (h + 1) * dk][free] *= 3.0
            proj[0, nq + h * dk:nq + (h + 1) * dk][free] = proj[1, nq + h * dk:nq + (h + 1) * dk][free]
        for h in range(heads):
            g = h // per
            proj[T - 1, h * dk:(h + 1) * dk][free] = proj[1, nq + g * dk:nq + (g + 1) * dk][free] * 1.5
    p32 = f32_round(proj)
    q = p32[:, :nq].reshape(T, heads, dk)
    k = p32[:, nq:nq + nk].reshape(T, kv, dk)
    v = k.copy() if from_keys else p32[:, nq + nk:nq + nk + nv].reshape(T, kv, dv)
    if normed:
        q, k = plain.rms_norm(q, f32_round(q_w), 1e-5), plain.rms_norm(k, f32_round(k_w), 1e-5)
    rot = dict(base=300.0, dims=rot_dims)
    pos = np.arange(T, dtype=np.int32)
    qn, kn = plain.rotate_half(q, pos, rot), plain.rotate_half(k, pos, rot)
    inv, tab = rotation_inputs(rot, 100)                      # beyond the table the angle is taken in 32-bit on the device
    table, n_pages = paged(rng, T, P)
    pool = torch.full((n_pages, kv, P, dk + dv), float("nan"), device="cuda", dtype=DT[dtype])
    q_out = torch.empty(T, nq, device="cuda", dtype=DT[dtype])
    slots = np.zeros(T, dtype=np.int32)
    cols = (0, nq, -1 if from_keys else nq + nk)
    for lo, hi in ((0, 37), (37, T - 1), (T - 1, T)):
        ops.gated_qkv_prep(dev(proj[lo:hi]), None if q_w is None else dev(q_w), None if k_w is None else dev(k_w), inv, tab,
                           dev(pos[lo:hi], torch.int32), dev(slots[lo:hi], torch.int32), dev(table, torch.int32), pool, q_out[lo:hi],
                           heads, kv, dk, dv, cols, eps=1e-5, rot_dims=rot_dims)
    tol = 1e-4 if dtype == "float32" else 2.0 ** -7
    assert np.abs(f64(q_out).reshape(T, heads, dk) - qn).max() < tol * max(1.0, np.abs(qn).max())
    flat = f64(pool).reshape(n_pages, -1)
    for t in (0, 1, P - 1, P, 36, 37, T - 2, T - 1):
        pg = flat[table[0, t // P]]
        keys = pg[:kv * P * dk].reshape(kv, P, dk)[:, t % P]
        vals = pg[kv * P * dk:].reshape(kv, dv, P)[:, :, t % P]
        assert np.abs(keys - kn[t]).max() < tol * max(1.0, np.abs(kn).max()), t
        assert np.abs(vals - v[t]).max() < tol * max(1.0, np.abs(v).max()), t
    if dtype == "bfloat16":
        qn, kn, v = bf16_round(qn), bf16_round(kn), bf16_round(v)
    sinks = rng.normal(0.5, 1.0, size=heads) if sink else None
    want = plain.softmax_heads(qn, kn, v, scale, None if sinks is None else f32_round(sinks))
    if free is not None and not normed:
        p_last = plain.causal_softmax(qn[:, 0] @ kn[:, 0].T * scale, None if sinks is None else float(f32_round(sinks)[0]))[T - 1]
        assert p_last[0] + p_last[1] > 0.2                    # the far keys matter
    gates = p32[:, nq + nk + nv + pad:]
    if gate == 1:
        want = want * plain.sigmoid(gates).reshape(T, heads, dv)
    elif gate == 2:
        want = want * plain.sigmoid(gates)[:, :, None]
    out = torch.empty(T, heads * dv, device="cuda", dtype=DT[dtype])
    ops.gated_attention(q_out, pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32),
                        None if sinks is None else dev(sinks), dev(proj) if gate else None, out, heads, kv, dk, dv, scale,
                        gate_col=nq + nk + nv + pad, gate_mode=gate)
    bound = 3e-5 if dtype == "float32" else 2e-2
    err = np.abs(f64(out).reshape(T, heads, dv) - want)
    assert err.max() < bound * max(1.0, np.abs(want).max()), (np.unravel_index(err.argmax(), err.shape), err.max())
    if sink:                                                  # without the sink the first rows come out differently
        ops.gated_attention(q_out, pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32), None,
                            dev(proj) if gate else None, out, heads, kv, dk, dv, scale, gate_col=nq + nk + nv + pad, gate_mode=gate)
        assert np.abs(f64(out).reshape(T, heads, dv)[:3] - want[:3]).max() > 10 * bound * np.abs(want[:3]).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv,dk,dv", [(4, 2, 64, 48), (2, 1, 32, 8), (3, 3, 128, 100)])
def test_values_padded_to_the_keys_size_in_the_pages(ops, dtype, heads, kv, dk, dv):
    """Pages with room for values of the keys' size: the rows beyond the value's size are written as zeros, and the attention
    over them gives the bits it gives over pages without the padding."""
    rng = np.random.default_rng(dk + dv)
    T, P = 75, 16
    nq, nk, nv = heads * dk, kv * dk, kv * dv
    proj = rng.normal(size=(T, nq + nk + nv + heads * dv))
    sink = dev(rng.normal(0.5, 1.0, size=heads))
    table, n_pages = paged(rng, T, P)
    pos, slots = np.arange(T, dtype=np.int32), np.zeros(T, dtype=np.int32)
    args = (dev(pos, torch.int32), dev(slots, torch.int32), dev(table, torch.int32))
    outs = []
    for rows in (dv, dk):
        pool = torch.full((n_pages, kv, P, dk + rows), float("nan"), device="cuda", dtype=DT[dtype])
        q_out = torch.empty(T, nq, device="cuda", dtype=DT[dtype])
        ops.gated_qkv_prep(dev(proj), None, None, None, None, *args, pool, q_out, heads, kv, dk, dv, (0, nq, nq + nk))
        flat = f64(pool).reshape(n_pages, -1)
        for t in (0, P - 1, P, T - 1):
            vals = flat[table[0, t // P]][kv * P * dk:].reshape(kv, rows, P)[:, :, t % P]
            want = f32_round(proj[t, nq + nk:nq + nk + nv]).reshape(kv, dv)
            if dtype == "bfloat16":
                want = bf16_round(want)
            assert np.array_equal(vals[:, :dv], want) and not vals[:, dv:].any(), t
        out = torch.empty(T, heads * dv, device="cuda", dtype=DT[dtype])
        ops.gated_attention(q_out, pool, args[2], args[0], args[1], sink, dev(proj), out, heads, kv, dk, dv, 0.2, gate_col=nq + nk + nv,
                            gate_mode=1)
        outs.append(f64(out))
    assert np.isfinite(outs[0]).all() and np.array_equal(outs[0], outs[1])


def test_values_mixed_with_the_first_layers(ops):
    """Mode 1 keeps the step's values as they are projected; mode 2 caches (1 - l) v + l kept, in 32-bit."""
    rng = np.random.default_rng(11)
    T, heads, kv, dk, dv, P = 21, 2, 2, 8, 12, 4
    nq, nk, nv = heads * dk, kv * dk, kv * dv
    first, later = rng.normal(size=(T, nq + nk + nv)), rng.normal(size=(T, nq + nk + nv))
    table, n_pages = paged(rng, T, P)
    pos, slots = np.arange(T, dtype=np.int32), np.zeros(T, dtype=np.int32)
    kept = torch.zeros(T, nv, device="cuda")
    q_out = torch.empty(T, nq, device="cuda")
    pools = [torch.zeros(n_pages, kv, P, dk + dv, device="cuda") for _ in range(2)]
    lam = 0.375
    args = (dev(pos, torch.int32), dev(slots, torch.int32), dev(table, torch.int32))
    ops.gated_qkv_prep(dev(first), None, None, None, None, *args, pools[0], q_out, heads, kv, dk, dv, (0, nq, nq + nk), mix_mode=1, kept=kept)
    assert np.array_equal(f64(kept), f32_round(first[:, nq + nk:]))
    ops.gated_qkv_prep(dev(later), None, None, None, None, *args, pools[1], q_out, heads, kv, dk, dv, (0, nq, nq + nk), mix_mode=2,
                       mix_lambda=dev([lam]), kept=kept)
    want = (1 - lam) * f32_round(later[:, nq + nk:]) + lam * f32_round(first[:, nq + nk:])
    for layer, ref in ((0, f32_round(first[:, nq + nk:])), (1, want)):
        flat = f64(pools[layer]).reshape(n_pages, -1)
        for t in range(T):
            vals = flat[table[0, t // P]][kv * P * dk:].reshape(kv, dv, P)[:, :, t % P]
            assert np.abs(vals.reshape(-1) - ref[t]).max() < 1e-6, (layer, t)


@pytest.mark.parametrize("heads,dk,dv", [(3, 8, 12), (1, 5, 7), (6, 32, 32), (2, 64, 64), (2, 128, 128), (1, 256, 64), (1, 200, 256)])
def test_decayed_linear_attention(ops, heads, dk, dv):
    """The scan over a request's tokens whole, in portions down to single tokens, and beside another request; the state in
    its slot carries from step to step; a slot that is zeroed serves the next request.  Cuts agree bit for bit."""
    rng = np.random.default_rng(dk + dv)
    T = 90
    nq, nv = heads * dk, heads * dv
    proj = rng.normal(size=(T, 2 * nq + nv + 4)) * 0.8
    decay = np.concatenate([[0.999], rng.uniform(0.3, 0.99, size=heads)])[:heads]
    p32, d32 = f32_round(proj), f32_round(decay)
    q = plain.silu(p32[:, 2:2 + nq]).reshape(T, heads, dk)
    k = plain.silu(p32[:, 2 + nq:2 + 2 * nq]).reshape(T, heads, dk)
    v = plain.silu(p32[:, 4 + 2 * nq:]).reshape(T, heads, dv)
    want = np.zeros((T, heads, dv))
    S = np.zeros((heads, dk, dv))
    for t in range(T):
        for h in range(heads):
            S[h] = d32[h] * S[h] + np.outer(k[t, h], v[t, h])
            want[t, h] = S[h].T @ q[t, h]
    cols = (2, 2 + nq, 4 + 2 * nq)
    state = torch.zeros(3, heads, dk * dv, device="cuda")
    state[1].fill_(float("nan"))                              # another request's slot: never touched
    pj, dc = dev(proj), dev(decay)

    def run(cuts, slot):
        o = torch.empty(T, nv, device="cuda")
        at = 0
        for n in cuts:
            ops.decay_scan(pj[at:at + n], dc, state, dev([[0, n, at, slot]], torch.int32), o[at:at + n], heads, dk, dv, cols)
            at += n
        assert at == T
        return f64(o).reshape(T, heads, dv)

    whole = run([T], 0)
    scale = np.abs(want).max()
    assert np.abs(whole - want).max() < 2e-5 * scale
    assert np.abs(f64(state[0]).reshape(heads, dk, dv) - S).max() < 2e-5 * np.abs(S).max()
    cut = run([17, 1, 1, 2, 33, 16, 1, 19], 2)
    assert np.array_equal(cut, whole)
    assert np.array_equal(f64(state[2]), f64(state[0]))
    state[0].zero_()                                          # the slot goes to the next request
    again = run([1] * 5 + [T - 5], 0)
    assert np.array_equal(again, whole)
    # the tokens in chunks that run side by side, the state carried from chunk to chunk: the same values up to rounding, and
    # the state behind them in the slot; a second step goes on from it token by token
    state[0].zero_()
    o = torch.empty(T, nv, device="cuda")
    sizes = [32, 32, 6]
    chunks = [[0, sum(sizes[:c]), n, (1 if c == 0 else 0) | (2 if c == len(sizes) - 1 else 0)] for c, n in enumerate(sizes)]
    ops.decay_scan(pj[:70], dc, state, dev([[0, 70, 0, 0]], torch.int32), o[:70], heads, dk, dv, cols, dev(chunks, torch.int32),
                   dev([[0, 3]], torch.int32))
    ops.decay_scan(pj[70:], dc, state, dev([[0, T - 70, 70, 0]], torch.int32), o[70:], heads, dk, dv, cols)
    assert np.abs(f64(o).reshape(T, heads, dv) - want).max() < 2e-5 * scale
    assert np.abs(f64(state[0]).reshape(heads, dk, dv) - S).max() < 2e-5 * np.abs(S).max()
    # two requests in one step, the second starting in the middle of the rows
    state[0].zero_()
    state[2].zero_()
    o = torch.empty(T, nv, device="cuda")
    both = torch.cat([pj[:40], pj[:50]])
    ops.decay_scan(both, dc, state, dev([[0, 40, 0, 2], [40, 50, 0, 0]], torch.int32), o, heads, dk, dv, cols)
    assert np.array_equal(f64(o[:40]).reshape(40, heads, dv), whole[:40]) and np.array_equal(f64(o[40:]).reshape(50, heads, dv), whole[:50])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_norm_over_all_heads(ops, dtype):
    rng = np.random.default_rng(5)
    M, W = 23, 84
    o = rng.normal(size=(M, W)) * np.linspace(0.1, 5.0, W)    # heads of very different size: a norm per head would show
    proj = rng.normal(size=(M, W + 9))
    w = rng.normal(1.0, 0.3, size=W)
    want = plain.rms_norm(f32_round(o), f32_round(w), 1e-5) * plain.sigmoid(f32_round(proj[:, 9:]))
    out = torch.empty(M, W, device="cuda", dtype=DT[dtype])
    ops.gated_row_norm(dev(o), dev(proj), 9, dev(w), 1e-5, out)
    assert np.abs(f64(out) - want).max() < (3e-5 if dtype == "float32" else 2.0 ** -7) * np.abs(want).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("E,top,groups,keep,W", [(6, 2, 3, 1, 40), (8, 3, 4, 2, 64), (5, 2, 5, 3, 50), (1, 1, 0, 0, 33), (12, 4, 1, 1, 128),
                                                 (16, 2, 2, 1, 96)])
def test_grouped_router(ops, dtype, E, top, groups, keep, W):
    rng = np.random.default_rng(E * 10 + top)
    M = 64
    h = rng.normal(size=(M, W))
    router = rng.normal(size=(E, W)) * 2.0 / math.sqrt(W)
    corr = rng.normal(0.0, 0.4, size=E) - 1.5                 # choice scores below zero: masked means minus infinity, not zero
    hq = bf16_round(h) if dtype == "bfloat16" else f32_round(h)
    w = {"m.router": f32_round(router), "m.correction": f32_round(corr)}
    r = dict(experts=E, top=top, scale=2.5)
    if groups:
        r["groups"] = dict(count=groups, keep=keep)
    ids_want, wts_want = plain.route(hq, r, w, "m")
    ids = torch.empty(M, top, device="cuda", dtype=torch.int32)
    wts = torch.empty(M, top, device="cuda")
    ops.moe_route_grouped(dev(h, DT[dtype]), dev(router), ids, wts, dev(corr), top, groups, keep, 2.5, 1e-20)
    # a choice within rounding of a tie may fall either way: such rows are left out (few), all others agree exactly
    s = plain.sigmoid(hq @ w["m.router"].T) + w["m.correction"]
    gap = np.array([np.min(np.abs(np.subtract.outer(s[t], s[t])[~np.eye(E, dtype=bool)])) if E > 1 else 1.0 for t in range(M)])
    sure = gap > 1e-4
    assert sure.mean() > 0.8
    assert np.array_equal(ids.cpu().numpy()[sure], ids_want[sure])
    assert np.abs(f64(wts)[sure] - wts_want[sure]).max() < 1e-5


def test_equal_choice_scores_go_to_the_lower_index_and_group(ops):
    W, E = 16, 8
    h = torch.zeros(3, W, device="cuda")                      # every score is 1/2
    ids = torch.empty(3, 2, device="cuda", dtype=torch.int32)
    wts = torch.empty(3, 2, device="cuda")
    ops.moe_route_grouped(h, torch.ones(E, W, device="cuda"), ids, wts, torch.zeros(E, device="cuda"), 2, 4, 2, 3.0, 1e-20)
    assert ids.cpu().tolist() == [[0, 1]] * 3 and np.abs(f64(wts) - 1.5).max() < 1e-6
    corr = torch.tensor([0, 0, 0, 0, 0.0, 0.0, 0.25, 0.25], device="cuda")      # the last group wins, then the lowest of the rest
    ids = torch.empty(3, 3, device="cuda", dtype=torch.int32)
    wts = torch.empty(3, 3, device="cuda")
    ops.moe_route_grouped(h, torch.ones(E, W, device="cuda"), ids, wts, corr, 3, 4, 2, 1.0, 1e-20)
    assert ids.cpu().tolist() == [[6, 7, 0]] * 3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gelu_gate(ops, dtype):
    rng = np.random.default_rng(9)
    z = rng.normal(size=(31, 2 * 45)) * 3
    out = torch.empty(31, 45, device="cuda", dtype=DT[dtype])
    ops.gated_act(dev(z), None, out, "gelu_tanh")
    z32 = f32_round(z)
    want = plain.gelu_tanh(z32[:, :45]) * z32[:, 45:]
    assert np.abs(f64(out) - want).max() < (2e-5 if dtype == "float32" else 2.0 ** -7) * np.abs(want).max()


# ---------------------------------------------------------------------------------- the engine
REQUEST_LENGTHS = {"a": 97, "b": 45, "c": 130, "d": 33, "e": 71, "f": 58}
PROMPT_LENGTHS = {"a": 60, "b": 12, "c": 101, "d": 30, "e": 2, "f": 41}
_made = {}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    def get(name):
        if name not in _made:
            config = dm.CONFIGS[name]
            weights = dm.draw_weights(config, seed=len(name) * 13 + 2)
            path = dm.write_folder(str(tmp_path_factory.mktemp("dubozen_" + name)), config, 0, weights)
            requests = {r: random_tokens(n, config["vocab"], 17 + i) for i, (r, n) in enumerate(REQUEST_LENGTHS.items())}
            w = dm.as_float64(weights)
            want = {r: plain.forward(config, w, t) for r, t in requests.items()}
            _made[name] = (path, requests, want, w)
        return _made[name]
    return get


def build_engine(folder, dtype, max_tokens, page_size=16, max_requests=4):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.engine import Engine
    return Engine.from_folder(folder, dtype, page_size=page_size, max_tokens=max_tokens, max_requests=max_requests, max_seq=max_tokens)


def replay(engine, trace):
    from tinyinfer_amd.engine import StepEntry
    got = {}
    for step in trace:
        logits = engine.step([StepEntry(r, t, w) for r, t, w in step["entries"]])
        rows = None if logits is None else logits.cpu().numpy().astype(np.float64)
        i = 0
        for r, _, w in step["entries"]:
            for _ in w:
                got.setdefault(r, []).append(rows[i])
                i += 1
        for r in step["end"]:
            engine.release(r)
        engine.cache.check()
    return {r: np.stack(v) for r, v in got.items()}


def errors(got, want):
    assert got.shape == want.shape, (got.shape, want.shape)
    d = got - want
    d = d - d.mean(axis=1, keepdims=True)
    ref = want - want.mean(axis=1, keepdims=True)
    return np.sqrt((d ** 2).mean(axis=1)) / np.sqrt((ref ** 2).mean(axis=1))


def worst(got, want):
    w, where = 0.0, None
    for r in want:
        e = errors(got[r], want[r])
        if e.max() > w:
            w, where = float(e.max()), (r, int(e.argmax()))
    return w, where


def within(got, want, dtype):
    """32-bit: every position within the bound.  bfloat16: all but 8 % of them, and the median far below it."""
    if dtype == "float32":
        w, where = worst(got, want)
        return w < TOL[dtype], (w, where)
    e = np.concatenate([errors(got[r], want[r]) for r in want])
    over = float((e > TOL[dtype]).mean())
    return over <= 0.08 and float(np.median(e)) < 2e-2, (over, float(np.median(e)), float(e.max()))


def make_trace(mode, requests):
    if mode == "whole":
        return traces.whole(requests)
    if mode == "tail":
        return traces.tail_one_by_one(requests, 32)
    if mode == "portions":
        return traces.portions(requests)
    return traces.mixed(requests, PROMPT_LENGTHS, live=4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,page_size", [("streams", 8), ("plain", 4), ("wide", 16), ("single", 16), ("squares", 16)])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_engine_matches_plain(folders, name, page_size, dtype, mode):
    folder, requests, want, _ = folders(name)
    trace = make_trace(mode, requests)
    n_tok = traces.max_pages(trace, page_size) * page_size      # the tightest pool: pages are handed out again
    engine = build_engine(folder, dtype, n_tok, page_size)       # four state slots for six requests: slots are used again
    got = replay(engine, trace)
    assert not engine.cache.live_requests()
    ok, seen = within(got, want, dtype)
    assert ok, (name, mode, dtype, seen)


@pytest.mark.parametrize("name", ["streams", "plain"])
def test_cuts_agree_bit_for_bit_in_float32(folders, name):
    """Token by token from the first token on, in portions, and whole: in 32-bit every sum is taken in an order that does
    not depend on the step, so the logits are the same bits."""
    folder, requests, _, _ = folders(name)
    some = {r: requests[r][:40] for r in ("b", "d")}
    results = []
    for trace in (traces.whole(some), traces.tail_one_by_one(some, 39), traces.portions(some), traces.mixed(some, {"b": 20, "d": 3}, live=2)):
        engine = build_engine(folder, "float32", 256)
        results.append(replay(engine, trace))
    for other in results[1:]:
        for r in some:
            assert np.array_equal(results[0][r], other[r]), r


def test_pages_and_slots_used_again_hold_nothing_of_their_last_owner(folders):
    """One request at a time in the smallest pool that holds it and one state slot: the second gets the pages and the slot
    the first gave back, and must find an empty memory there."""
    folder, requests, want, _ = folders("streams")
    engine = build_engine(folder, "float32", 144, page_size=8, max_requests=1)
    for r in ("c", "b", "c"):
        got = replay(engine, traces.portions({r: requests[r]}))
        w, where = worst(got, {r: want[r]})
        assert w < TOL["float32"], (r, w, where)


def test_long_decoding(folders):
    """A prompt of 50 tokens in portions of 32, then 250 tokens one by one: the state of the linear attention is carried through
    every step, and the keys of the first tokens stay visible to the last."""
    from tinyinfer_amd.engine import StepEntry
    folder, _, _, w = folders("streams")
    config = dm.CONFIGS["streams"]
    toks = random_tokens(300, config["vocab"], 99)
    want = plain.forward(config, w, toks)
    for dtype in ("float32", "bfloat16"):
        engine = build_engine(folder, dtype, 320, page_size=8)
        rows, at = [], 0
        while at < 50:
            n = min(32, 50 - at)
            rows.append(engine.step([StepEntry("x", toks[at:at + n], list(range(n)))]).cpu().numpy())
            at += n
        for t in toks[50:]:
            rows.append(engine.step([StepEntry("x", [t], [0])]).cpu().numpy())
            engine.cache.check()
        got = np.concatenate(rows).astype(np.float64)
        ok, seen = within({"x": got}, {"x": want}, dtype)
        assert ok, (dtype, seen)


def test_a_token_far_back_reaches_the_last_position(folders):
    """Changing token 3 of 120 moves the last position's logits, through the cached keys and through the carried state alike
    (the plain model says by how much; the engine, fed in a portion and then token by token, agrees with it)."""
    from tinyinfer_amd.engine import StepEntry
    folder, requests, _, w = folders("streams")
    config = dm.CONFIGS["streams"]
    toks = list(requests["c"][:120])
    other = list(toks)
    other[3] = (other[3] + 1) % config["vocab"]
    engine = build_engine(folder, "float32", 256, page_size=8)
    outs = []
    for i, t in enumerate((toks, other)):
        engine.step([StepEntry(str(i), t[:100], [])])
        for tok in t[100:119]:
            engine.step([StepEntry(str(i), [tok], [])])
        outs.append(engine.step([StepEntry(str(i), [t[119]], [0])]).cpu().numpy()[0].astype(np.float64))
        engine.release(str(i))
    want = [plain.forward(config, w, t)[-1] for t in (toks, other)]
    assert np.abs(want[0] - want[1]).max() > 1e-3
    for g, wnt in zip(outs, want):
        assert errors(g[None], wnt[None])[0] < TOL["float32"]


@pytest.mark.parametrize("use_graph", [False, True])
def test_greedy_generation_through_the_entry_point(folders, use_graph):
    """Several prompts of unequal length at once through LLM.generate: the scheduler cuts the prompts into portions of 16
    and batches decoding requests; every generated token is the plain model's argmax."""
    import tinyinfer_amd as ti
    folder, requests, _, w = folders("streams")
    config = dm.CONFIGS["streams"]
    prompts = [requests["b"][:37], requests["d"][:5], requests["e"][:50], requests["f"][:1]]
    n_new = 12
    llm = ti.LLM(folder, dtype="float32", max_seq=128, max_requests=3, chunk_size=16, max_batched_tokens=40, use_graph=use_graph)
    got = llm.generate(prompts, max_new_tokens=n_new, temperature=0.0)
    for p, g in zip(prompts, got):
        toks = list(p)
        for _ in range(n_new):
            logits = plain.forward(config, w, toks)[-1]
            best = int(np.argmax(logits))
            margin = logits[best] - np.partition(logits, -2)[-2]
            toks.append(best)
            if margin < 1e-3:          # a tie within rounding: what follows may differ legitimately
                break
        n = len(toks) - len(p)
        assert g[:n] == toks[len(p):], (p[:3], g, toks[len(p):])


def test_graphs_replay_the_bfloat16_kernels(folders):
    """bfloat16 at sizes the matrix cores serve: decoding from captured graphs gives the tokens that decoding step by step gives."""
    import tinyinfer_amd as ti
    folder, requests, _, _ = folders("wide")
    prompts = [requests["b"][:37], requests["d"][:5], requests["e"][:50]]
    outs = []
    for use_graph in (False, True):
        llm = ti.LLM(folder, dtype="bfloat16", max_seq=128, max_requests=3, chunk_size=32, max_batched_tokens=64, use_graph=use_graph)
        outs.append(llm.generate(prompts, max_new_tokens=20, temperature=0.0))
    assert outs[0] == outs[1]


def test_matrix_core_attention_takes_the_sink_where_it_finishes_a_column(tmp_path):
    """bfloat16 at keys and values of 64: a long prompt whole (tiles, in pairs and one by one), then single tokens with every
    context split over workgroups and not split.  Every way agrees with the row-wise kernels and with the plain model; with
    the sinks taken out of the weights the logits move, so the agreement is not of models that ignore them."""
    from tinyinfer_amd.engine import StepEntry
    config = dm.CONFIGS["wide"]
    weights = dm.draw_weights(config, seed=77)
    for k in weights:
        if k.endswith(".sink"):
            weights[k] = weights[k] + 3.0                 # sinks as heavy as dozens of keys together ...
        if k in ("l1.mix.o", "l2.mix.o"):
            weights[k] = weights[k] * 6.0                 # ... in layers that weigh much in the residual
    folder = dm.write_folder(str(tmp_path / "sinks"), config, 0, weights)
    w = dm.as_float64(weights)
    toks = random_tokens(420, config["vocab"], 5)
    want = plain.forward(config, w, toks)
    no_sink = dict(w)
    for k in w:
        if k.endswith(".sink"):
            no_sink[k] = w[k] - 30.0
    assert np.median(errors(plain.forward(config, no_sink, toks[:64]), want[:64])) > 0.15

    def run(fast, splits=0, paired=None):
        engine = build_engine(folder, "bfloat16", 448)
        engine.ops.use_fast_attention = fast
        engine.ops.force_decode_splits = splits
        engine.ops.force_paired_tiles = paired
        engine.ops.count_calls(True)
        rows = [engine.step([StepEntry("x", toks[:400], list(range(400)))]).cpu().numpy()]
        for t in toks[400:]:
            rows.append(engine.step([StepEntry("x", [t], [0])]).cpu().numpy())
        names = [r["name"] for r in engine.ops.timing_report()]
        engine.ops.count_calls(False)
        return np.concatenate(rows).astype(np.float64), names

    slow, names = run(False)
    assert any(n.startswith("gated_attention") and n.endswith("[generic]") for n in names)
    assert not any(n.endswith("[mfma]") and n.startswith("gated_attention") for n in names)
    ok, seen = within({"x": slow}, {"x": want}, "bfloat16")
    assert ok, seen
    for splits, paired in ((0, None), (4, True), (1, False)):
        fast, names = run(True, splits, paired)
        assert any(n.startswith("gated_attention") and n.endswith("[mfma]") for n in names), names
        ok, seen = within({"x": fast}, {"x": want}, "bfloat16")
        assert ok, (splits, paired, seen)
        e = errors(fast, slow)
        # a router's choice within rounding of a tie may fall the other way at a position or two
        assert np.median(e) < 2e-2 and (e > 0.08).mean() <= 0.05, (splits, paired, float(np.median(e)), float(e.max()))


def plain_greedy(config, w, prompt, n_new):
    """(generated ids, how many of them stand clear of a tie within rounding)."""
    toks, sure = list(prompt), 0
    for k in range(n_new):
        logits = plain.forward(config, w, toks)[-1]
        best = int(np.argmax(logits))
        if sure == k and logits[best] - np.partition(logits, -2)[-2] > 1e-3:
            sure = k + 1
        toks.append(best)
    return toks[len(prompt):], sure


def test_command_line_generates_from_a_dubozen_folder(folders):
    """bin/tinyinfer picks the model by config.json: token ids in, the plain model's greedy tokens out; with --cuda-graph too."""
    import os
    import subprocess
    import sys
    folder, requests, _, w = folders("plain")
    config = dm.CONFIGS["plain"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p1, p2 = requests["b"][:11], requests["d"][:4]
    for extra in ([], ["--cuda-graph"]):
        run = subprocess.run([sys.executable, os.path.join(root, "bin", "tinyinfer"), "-m", folder, "-n", "6", "-p", ",".join(map(str, p1)),
                              "-p", " ".join(map(str, p2)), "--dtype", "float32", "--max-seq", "64"] + extra,
                             capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr[-2000:]
        outputs = [l[len("[output] "):].split() for l in run.stdout.split("\n") if l.startswith("[output] ")]
        assert len(outputs) == 2
        for p, got in zip((p1, p2), outputs):
            want, sure = plain_greedy(config, w, p, 6)
            assert [int(t) for t in got][:sure] == want[:sure], (got, want)


def test_random_weights_drawn_on_the_device_run():
    """A config.json alone: the parts' declared distributions give a model that steps (what the bench tool measures)."""
    from tinyinfer_amd.engine import Engine, StepEntry
    for name in ("streams", "wide"):
        engine = Engine.from_config(dm.CONFIGS[name], seed=3, dtype="bfloat16", page_size=16, max_tokens=256, max_requests=2, max_seq=256)
        toks = random_tokens(70, dm.CONFIGS[name]["vocab"], 1)
        a = engine.step([StepEntry("x", toks, [69])]).cpu().numpy()
        engine.release("x")
        assert engine.step([StepEntry("y", toks[:69], [])]) is None
        b = engine.step([StepEntry("y", toks[69:], [0])]).cpu().numpy()
        assert np.isfinite(a).all() and a.std() > 0
        assert np.abs(a - b).max() < 0.08 * max(1e-6, np.abs(a).max())


def test_trace_replay_program(folders, tmp_path):
    """The replay program on a Dubozen folder: it picks the model by config.json and writes the logits the engine gives."""
    import os
    import subprocess
    import sys
    folder, requests, want, _ = folders("plain")
    some = {r: requests[r] for r in ("b", "d", "f")}
    trace = traces.mixed(some, PROMPT_LENGTHS, live=2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", str(traces.max_tokens(trace))], input=traces.to_jsonl(trace), text=True,
                          capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    V = dm.CONFIGS["plain"]["vocab"]
    got = {}
    for i, step in enumerate(trace):
        assert f"done {i}" in proc.stdout
        rows = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V).astype(np.float64)
        k = 0
        for r, _, wnt in step["entries"]:
            for _ in wnt:
                got.setdefault(r, []).append(rows[k])
                k += 1
    w, where = worst({r: np.stack(v) for r, v in got.items()}, {r: want[r] for r in some})
    assert w < TOL["float32"], (w, where)
