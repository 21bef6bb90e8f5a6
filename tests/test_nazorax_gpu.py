"""Nazorax on the GPU against the plain implementation: every mechanism alone through the kernels' own object, and the
engine under every way of cutting the work (each request whole; most of it in one step and its last tokens one by
one; portions of changing size down to two tokens; up to four live requests mixed, with so few pages that they are
used again), in 32-bit and in bfloat16, and greedy generation through the entry point and the scheduler."""
import math

import numpy as np
import pytest
import torch

import nazorax_models as nm
import traces
from helpers import random_tokens
from plain import nazorax_plain as plain

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# rms of (engine - plain) over rms of the plain logits, per position.  float32: rounding of 32-bit sums against float64.
# bfloat16: operands of every product, cached keys, values and latents and the queries are rounded to 8 bits, which moves
# the logits by a per cent or two, while a lost key, a window that is one token off, a forgotten sink or a wrong expert
# moves them by tens of per cent.  Where two experts' logits lie within that rounding of each other, bfloat16 may pick the
# other one with nothing wrong: in bfloat16 the bound holds for all but 8 % of the positions and the median error stays
# under 2 %; 32-bit holds everywhere.
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


def paged(rng, n_tokens, P, extra_pages=3):
    n_pages = -(-n_tokens // P)
    ids = rng.permutation(n_pages + extra_pages)[:n_pages]
    return np.asarray(ids, dtype=np.int32)[None, :], n_pages + extra_pages


# ---------------------------------------------------------------------------------- each mechanism alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("W", [50, 192, 1030])
def test_dynamic_tanh(ops, dtype, W):
    rng = np.random.default_rng(W)
    x = rng.normal(size=(7, W)) * 2
    w = {"n": 1.0 + rng.normal(size=W) * 0.3, "n.b": rng.normal(size=W), "n.alpha": np.asarray(0.6)}
    want = plain.dynamic_tanh(x.astype(np.float32).astype(np.float64), w, "n")
    tol = 3e-6 if dtype == "float32" else 2.0 ** -7
    out = torch.empty(7, W, device="cuda", dtype=DT[dtype])
    ops.dyt(dev(x), dev([0.6]), dev(w["n"]), dev(w["n.b"]), out)
    assert np.abs(f64(out) - want).max() < tol * max(1.0, np.abs(want).max())
    rows = [5, 0, 5, 2]                                     # the wanted rows only, one of them twice
    out = torch.empty(4, W, device="cuda", dtype=DT[dtype])
    ops.dyt(dev(x), dev([0.6]), dev(w["n"]), dev(w["n.b"]), out, dev(rows, torch.int32))
    assert np.abs(f64(out) - want[rows]).max() < tol * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("F", [9, 64, 130])
def test_gated_activations(ops, dtype, F):
    rng = np.random.default_rng(F)
    z = rng.normal(size=(6, 2 * F)) * 3                     # many entries beyond the limits
    b = rng.normal(size=2 * F)
    tol = 3e-6 if dtype == "float32" else 2.0 ** -7
    z32 = z.astype(np.float32).astype(np.float64)
    out = torch.empty(6, F, device="cuda", dtype=DT[dtype])
    ops.gated_act(dev(z), dev(b), out, "silu")
    g, u = z32[:, :F] + b.astype(np.float32)[:F], z32[:, F:] + b.astype(np.float32)[F:]
    want = plain.silu(g) * u
    assert np.abs(f64(out) - want).max() < tol * max(1.0, np.abs(want).max())
    for limit in (0.7, 2.5):
        ops.gated_act(dev(z), None, out, "clamped", limit)
        g, u = np.minimum(z32[:, :F], limit), np.clip(z32[:, F:], -limit, limit)
        want = g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)
        assert np.abs(f64(out) - want).max() < tol * max(1.0, np.abs(want).max())


def test_two_streams_side_by_side(ops):
    rng = np.random.default_rng(3)
    for W in (50, 64):
        a, b = rng.normal(size=(5, W)).astype(np.float32), rng.normal(size=(5, W)).astype(np.float32)
        for dtype in ("float32", "bfloat16"):
            out = torch.empty(5, 2 * W, device="cuda", dtype=DT[dtype])
            ops.concat_round(dev(a), dev(b), out)
            assert torch.equal(out, torch.cat([dev(a), dev(b)], dim=1).to(DT[dtype]))


def rotation_inputs(rot, n_table):
    """(inv_freq, table of the first n_table positions, factor on cos and sin) as the kernels take them."""
    if not rot["dims"]:
        return None, None, 1.0
    freq, mag = plain.frequencies(rot)
    ang = np.arange(n_table)[:, None] * freq[None, :]
    return dev(freq), dev(np.stack([np.cos(ang) * mag, np.sin(ang) * mag], axis=-1)), mag


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv,dk,dv,P,window,rot_dims", [(4, 2, 16, 24, 16, 40, 8), (3, 3, 7, 9, 4, 13, 6), (6, 1, 40, 33, 64, 129, 40),
                                                               (2, 2, 64, 64, 16, 64, 32), (2, 1, 64, 32, 16, 0, 0), (3, 1, 24, 16, 8, 1, 12),
                                                               (8, 2, 128, 128, 32, 47, 64), (2, 2, 32, 32, 16, 33, 32)])
def test_biased_rotated_window_attention(ops, dtype, heads, kv, dk, dv, P, window, rot_dims):
    """q/k/v of a whole request get their biases, the rotation of their first entries, and go into the pages in two portions;
    then the attention of every row.  On the entries that are not rotated the last row's query points at the oldest key
    the window keeps, and the key just behind it is as strong: losing the first or seeing the second shows."""
    rng = np.random.default_rng(dk * 1000 + dv)
    T = 150
    scale = 1.3 / math.sqrt(dk)
    per = heads // kv
    q = rng.normal(size=(T, heads, dk))
    k = rng.normal(size=(T, kv, dk))
    v = rng.normal(size=(T, kv, dv))
    bias = rng.normal(size=heads * dk + kv * dk + kv * dv) * 0.5
    rot = dict(base=300.0, dims=rot_dims)
    inv, tab, mag = rotation_inputs(rot, 100)               # the rest take the angle in 32-bit on the device
    qkv = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], axis=1)
    b32 = bias.astype(np.float32).astype(np.float64)
    full = qkv.astype(np.float32).astype(np.float64) + b32
    qb = full[:, :heads * dk].reshape(T, heads, dk)
    kb = full[:, heads * dk:heads * dk + kv * dk].reshape(T, kv, dk)
    vb = full[:, heads * dk + kv * dk:].reshape(T, kv, dv)
    oldest = T - window if 0 < window < T else 0
    strong = rot_dims < dk and oldest > 0
    if strong:                                              # through the raw inputs, so that the kernel sees them
        group = np.arange(heads) // per
        for j in (oldest, oldest - 1):
            kb[j, :, rot_dims:] *= 4 if dk - rot_dims >= 4 else 12
        qb[T - 1, :, rot_dims:] = kb[oldest][group, rot_dims:] * (1 if dk - rot_dims >= 4 else 0.25)
        qkv = np.concatenate([qb.reshape(T, -1), kb.reshape(T, -1), vb.reshape(T, -1)], axis=1) - b32
        full = qkv.astype(np.float32).astype(np.float64) + b32
        qb = full[:, :heads * dk].reshape(T, heads, dk)
        kb = full[:, heads * dk:heads * dk + kv * dk].reshape(T, kv, dk)
    table, n_pages = paged(rng, T, P)
    pool = torch.zeros(n_pages, kv, P, dk + dv, device="cuda", dtype=DT[dtype])
    q_out = torch.empty(T, heads * dk, device="cuda", dtype=DT[dtype])
    pos = np.arange(T, dtype=np.int32)
    slots = np.zeros(T, dtype=np.int32)
    cut = 37
    for lo, hi in ((0, cut), (cut, T)):
        ops.qkv_prep_write(dev(qkv[lo:hi]), dev(bias), inv, tab, dev(pos[lo:hi], torch.int32), dev(slots[lo:hi], torch.int32),
                           dev(table, torch.int32), pool, q_out[lo:hi], heads, kv, dk, dv, rot_dims, mag)
    qn, kn = (plain.rotate_half(qb, pos, rot), plain.rotate_half(kb, pos, rot)) if rot_dims else (qb, kb)
    tol = 3e-5 if dtype == "float32" else 2.0 ** -7
    assert np.abs(f64(q_out).reshape(T, heads, dk) - qn).max() < tol * max(1.0, np.abs(qn).max())
    flat = f64(pool).reshape(n_pages, -1)
    for t in (0, 1, P - 1, P, cut - 1, cut, T - 1):
        pg = flat[table[0, t // P]]
        keys = pg[:kv * P * dk].reshape(kv, P, dk)[:, t % P]
        vals = pg[kv * P * dk:].reshape(kv, dv, P)[:, :, t % P]
        assert np.abs(keys - kn[t]).max() < tol * max(1.0, np.abs(kn).max()), t
        assert np.abs(vals - vb[t]).max() < tol * max(1.0, np.abs(vb).max()), t
    if dtype == "bfloat16":
        qn, kn, vb = bf16_round(qn), bf16_round(kn), bf16_round(vb)
    visible = plain.window_mask(T, window or None)
    want = np.zeros((T, heads, dv))
    for h in range(heads):
        p = plain.softmax_rows(qn[:, h] @ kn[:, h // per].T * scale, visible)
        want[:, h] = p @ vb[:, h // per]
        if strong and window > 1:
            assert p[T - 1, oldest] > 0.15                  # the oldest key the window keeps matters
    out = torch.empty(T, heads * dv, device="cuda", dtype=DT[dtype])
    ops.attention_capped(q_out, pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32), out, heads, kv, dk, dv,
                         scale, 0.0, window)
    bound = 2e-5 if dtype == "float32" else 2e-2
    err = np.abs(f64(out).reshape(T, heads, dv) - want)
    assert err.max() < bound * max(1.0, np.abs(want).max()), (np.unravel_index(err.argmax(), err.shape), err.max())


def latent_weights(rng, W, H, d, r, dv, R):
    w = {"m.q": rng.normal(size=(H * (d + r), W)) * 2 / math.sqrt(W), "m.dkv": rng.normal(size=(R + r, W)) * 2 / math.sqrt(W),
         "m.dkv.norm": 1.0 + rng.normal(size=R) * 0.3, "m.uk": rng.normal(size=(H * d, R)) * 1.5 / math.sqrt(R),
         "m.uv": rng.normal(size=(H * dv, R)) / math.sqrt(R), "m.sink": rng.normal(size=H) + 0.5, "m.o": np.eye(H * dv)}
    return {k: bf16_round(v) for k, v in w.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,d,r,dv,R,P,scaling", [(2, 12, 8, 10, 24, 8, True), (1, 2, 6, 7, 9, 4, True), (3, 8, 4, 16, 20, 16, False),
                                                   (4, 32, 16, 32, 64, 16, True), (5, 16, 0, 8, 40, 64, False), (2, 1, 8, 12, 16, 16, False),
                                                   (8, 64, 32, 64, 128, 16, True), (16, 128, 64, 128, 512, 16, True)])
def test_latent_attention_with_a_sink(ops, dtype, H, d, r, dv, R, P, scaling):
    """A whole request's projections prepared into the pages in two portions, then the attention of every row, against the
    mixer of the plain implementation (its output projection the identity).  An early token's input is made large: its
    latent loses that in its norm, its key part keeps it; a norm that is left out and a sink that is forgotten show.  (A far
    key and a window's edge that stand out: the test of the matrix-core kernels below, whose row-wise run reads the same pages.)"""
    rng = np.random.default_rng(H * 100 + R)
    T, W, eps = (150 if R < 512 else 70), 48, 1e-5
    m = dict(heads=H, dim=d, rot_dim=r, vdim=dv, kv_rank=R, scale=1.2 / math.sqrt(d + r),
             rot=dict(base=500.0, dims=r, scaling=nm.yarn(4.0, 32, 8.0, 1.0) if scaling and r else None))
    w = latent_weights(rng, W, H, d, r, dv, R)
    h = bf16_round(rng.normal(size=(T, W)))
    h[2] *= 6.0
    want = plain.latent_attention(h, w, "m", m, eps).reshape(T, H, dv)
    without_sink = plain.latent_attention(h, dict(w, **{"m.sink": np.full(H, -1e9)}), "m", m, eps).reshape(T, H, dv)
    assert np.abs(want - without_sink).max() > 0.05
    nq = H * (d + r)
    proj = h @ np.concatenate([w["m.q"], w["m.dkv"]]).T          # what the mixer's first product leaves, in 32-bit
    inv, tab, mag = rotation_inputs(m["rot"], 100) if r else (None, None, 1.0)
    table, n_pages = paged(rng, T, P)
    pool = torch.zeros(n_pages, P, R + r, device="cuda", dtype=DT[dtype])
    pos = np.arange(T, dtype=np.int32)
    slots = np.zeros(T, dtype=np.int32)
    pj = dev(proj)
    cut = 37
    for lo, hi in ((0, cut), (cut, T)):
        ops.latent_prep(pj[lo:hi], dev(w["m.dkv.norm"]), inv, tab, dev(pos[lo:hi], torch.int32), dev(slots[lo:hi], torch.int32),
                        dev(table, torch.int32), pool, nq, eps, H, d, r, R, r, mag)
    # what the pages hold: the normed latent and the rotated key part
    c = plain.rms_unit(proj[:, nq:nq + R], eps) * w["m.dkv.norm"]
    kr = plain.rotate_half(proj[:, nq + R:], pos, m["rot"]) if r else proj[:, nq + R:]
    flat = f64(pool).reshape(n_pages, P, R + r)
    tol = 3e-5 if dtype == "float32" else 2.0 ** -7
    for t in (0, 1, 2, P - 1, P, cut - 1, cut, T - 1):
        row = flat[table[0, t // P], t % P]
        assert np.abs(row[:R] - c[t]).max() < tol * max(1.0, np.abs(c).max()), t
        assert r == 0 or np.abs(row[R:] - kr[t]).max() < tol * max(1.0, np.abs(kr).max()), t
    out = torch.empty(T, H * dv, device="cuda", dtype=DT[dtype])
    ops.latent_attention(pj, dev(w["m.uk"], DT[dtype]), dev(w["m.uv"], DT[dtype]), dev(w["m.sink"]), pool, dev(table, torch.int32),
                         dev(pos, torch.int32), dev(slots, torch.int32), out, H, d, r, R, dv, m["scale"])
    bound = 1e-4 if dtype == "float32" else 4e-2
    err = np.abs(f64(out).reshape(T, H, dv) - want)
    assert err.max() < bound * max(1.0, np.abs(want).max()), (np.unravel_index(err.argmax(), err.shape), err.max())
    # single rows as decoded tokens: both sides of every page border, the first tokens, the last
    rows = sorted({0, 1, 2, P - 1, P, P + 1, 2 * P - 1, 2 * P, cut - 1, cut, T - 2, T - 1} & set(range(T)))
    for i in rows:
        one = torch.empty(1, H * dv, device="cuda", dtype=DT[dtype])
        ops.latent_attention(pj[i:i + 1], dev(w["m.uk"], DT[dtype]), dev(w["m.uv"], DT[dtype]), dev(w["m.sink"]), pool,
                             dev(table, torch.int32), dev(pos[i:i + 1], torch.int32), dev(slots[i:i + 1], torch.int32), one, H, d, r, R,
                             dv, m["scale"])
        err = np.abs(f64(one).reshape(H, dv) - want[i])
        assert err.max() < bound * max(1.0, np.abs(want).max()), (i, err.max())


@pytest.mark.parametrize("H,d,r,dv,R,P,window", [(4, 32, 16, 32, 64, 16, 0), (8, 64, 32, 64, 128, 16, 0), (16, 128, 64, 128, 512, 16, 0),
                                                  (3, 8, 8, 16, 16, 32, 0), (20, 24, 8, 48, 96, 16, 0), (2, 40, 24, 16, 240, 64, 0),
                                                  (6, 16, 48, 32, 112, 16, 50)])
def test_latent_attention_on_the_matrix_cores(ops, H, d, r, dv, R, P, window):
    """bfloat16, pages that hold the latents transposed as well: the request as one portion in tiles of 64 rows (the last one
    short), every row as a single token, some rows as tiles beside others as single tokens, and single tokens with their keys
    split over several workgroups, against the plain mixer; the row-wise kernels read the same pages."""
    rng = np.random.default_rng(H * 100 + R)
    T, W, eps = (150 if R < 512 else 100), 48, 1e-5
    m = dict(heads=H, dim=d, rot_dim=r, vdim=dv, kv_rank=R, scale=1.2 / math.sqrt(d + r),
             rot=dict(base=500.0, dims=r, scaling=nm.yarn(4.0, 32, 8.0, 1.0)))
    w = latent_weights(rng, W, H, d, r, dv, R)
    h = bf16_round(rng.normal(size=(T, W)))
    nq = H * (d + r)
    proj = h @ np.concatenate([w["m.q"], w["m.dkv"]]).T
    pos = np.arange(T, dtype=np.int32)
    # One key is made to stand out for the last row of every head, through the projections themselves: the oldest key the
    # window keeps (no window: the third token, far back among the others), and the key just behind the window gets the same
    # latent, so that losing the first or seeing the second shows.
    target = T - window if window else 2
    if window:
        proj[target - 1, nq:nq + R] = proj[target, nq:nq + R]
    c_all = plain.rms_unit(proj[:, nq:nq + R], eps) * w["m.dkv.norm"]
    for hd in range(H):                                     # the query: along the target's key, across what all keys share
        k_all = c_all @ w["m.uk"][hd * d:(hd + 1) * d].T
        dq = k_all[target] - k_all.mean(axis=0)
        proj[T - 1, hd * (d + r):hd * (d + r) + d] = dq * (14.0 / (dq @ k_all[target] * m["scale"]))
        proj[T - 1, hd * (d + r) + d:(hd + 1) * (d + r)] = 0.0
    proj = proj.astype(np.float32).astype(np.float64)
    inv, tab, mag = rotation_inputs(m["rot"], 100)
    table, n_pages = paged(rng, T, P)
    pool = torch.full((n_pages, P, 2 * R + r), float("nan"), device="cuda", dtype=torch.bfloat16)      # rows never written hold anything
    slots = np.zeros(T, dtype=np.int32)
    pj = dev(proj)
    cut = 37
    for lo, hi in ((0, cut), (cut, T)):
        ops.latent_prep(pj[lo:hi], dev(w["m.dkv.norm"]), inv, tab, dev(pos[lo:hi], torch.int32), dev(slots[lo:hi], torch.int32),
                        dev(table, torch.int32), pool, nq, eps, H, d, r, R, r, mag)
    flat = f64(pool).reshape(n_pages, -1)
    for t in (0, 1, P - 1, P, cut, T - 1):                  # the transposed latents are the rows' latents
        pg = flat[table[0, t // P]]
        assert np.array_equal(pg[:P * (R + r)].reshape(P, R + r)[t % P, :R], pg[P * (R + r):].reshape(R, P)[:, t % P]), t
    # the mixer's formulas on the projections, with what the pages hold rounded as the pages round it
    want = np.zeros((T, H, dv))
    q = proj[:, :nq].reshape(T, H, d + r)
    c = bf16_round(plain.rms_unit(proj[:, nq:nq + R], eps) * w["m.dkv.norm"])
    kr = bf16_round(plain.rotate_half(proj[:, nq + R:], pos, m["rot"]))
    qr = plain.rotate_half(q[:, :, d:], pos, m["rot"])
    vis = plain.window_mask(T, window or None)
    for hd in range(H):
        sc = (q[:, hd, :d] @ (c @ w["m.uk"][hd * d:(hd + 1) * d].T).T + qr[:, hd] @ kr.T) * m["scale"]
        p_att = plain.softmax_rows(sc, vis, float(w["m.sink"][hd]))
        assert (d < 16 or p_att[T - 1, target] > 0.2) and (not window or p_att[T - 1, target - 1] == 0.0)
        want[:, hd] = p_att @ (c @ w["m.uv"][hd * dv:(hd + 1) * dv].T)
    uk, uv = dev(w["m.uk"], torch.bfloat16), dev(w["m.uv"], torch.bfloat16)
    uk_t = torch.empty(H * R, d, device="cuda", dtype=torch.bfloat16)
    ops.latent_transpose(uk, uk_t, H)
    assert torch.equal(uk_t.reshape(H, R, d), uk.reshape(H, d, R).transpose(1, 2))
    args = (pj, uk, uv, dev(w["m.sink"]), pool, dev(table, torch.int32), dev(pos, torch.int32), dev(slots, torch.int32))
    sizes = (H, d, r, R, dv, m["scale"], window)
    bound = 4e-2 * max(1.0, np.abs(want).max())
    slow = torch.zeros(T, H * dv, device="cuda", dtype=torch.bfloat16)
    ops.latent_attention(*args, slow, *sizes)
    err = np.abs(f64(slow).reshape(T, H, dv) - want)
    assert err.max() < bound, ("rows", np.unravel_index(err.argmax(), err.shape), err.max())
    entries = dev([[0, T, 0, 0]], torch.int32)
    tiles = dev([[0, r0, min(64, T - r0)] for r0 in range(0, T, 64)], torch.int32)
    ops.count_calls(True)
    for lists in (dict(tiles=tiles, entries=entries), dict(all_rows=True), dict(all_rows=True, context=T),
                  dict(tiles=tiles[:1], entries=entries, rows=dev(list(range(64, T)), torch.int32))):
        fast = torch.zeros(T, H * dv, device="cuda", dtype=torch.bfloat16)
        ops.latent_attention(*args, fast, *sizes, w_uk_t=uk_t, **lists)
        err = np.abs(f64(fast).reshape(T, H, dv) - want)
        assert err.max() < bound, (list(lists), np.unravel_index(err.argmax(), err.shape), err.max())
    ops.force_decode_splits = 3
    fast = torch.zeros(T, H * dv, device="cuda", dtype=torch.bfloat16)
    ops.latent_attention(*args, fast, *sizes, w_uk_t=uk_t, all_rows=True, context=T)
    ops.force_decode_splits = 0
    err = np.abs(f64(fast).reshape(T, H, dv) - want)
    assert err.max() < bound, ("split", np.unravel_index(err.argmax(), err.shape), err.max())
    took = [c["name"] for c in ops.timing_report() if "latent_attention" in c["name"]]
    ops.count_calls(False)
    assert took and all("[mfma]" in n for n in took), took


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_router_over_the_chosen_and_clamped_experts(ops, dtype):
    rng = np.random.default_rng(11)
    # the last two: enough pairs for the grouped matrix-core path in bfloat16 (experts with no token, with one, with hundreds)
    for M, W, E, top, F, limit in [(9, 48, 5, 2, 40, 1.2), (3, 50, 1, 1, 9, 3.0), (17, 130, 70, 8, 33, 0.8), (4, 64, 8, 8, 64, 2.0),
                                   (300, 96, 11, 3, 160, 1.5), (200, 64, 40, 1, 32, 1.0)]:
        h = bf16_round(rng.normal(size=(M, W)))
        w = {"m.router": rng.normal(size=(E, W)).astype(np.float32).astype(np.float64) * 2 / math.sqrt(W)}
        w["m.router"] = w["m.router"].astype(np.float32).astype(np.float64)
        for e in range(E):
            w[f"m.e{e}.gate"] = bf16_round(rng.normal(size=(F, W)) * 2 / math.sqrt(W))
            w[f"m.e{e}.up"] = bf16_round(rng.normal(size=(F, W)) * 2 / math.sqrt(W))
            w[f"m.e{e}.down"] = bf16_round(rng.normal(size=(W, F)) / math.sqrt(F))
        ids = torch.empty(M, top, device="cuda", dtype=torch.int32)
        wts = torch.empty(M, top, device="cuda")
        ops.moe_route(dev(h, DT[dtype]), dev(w["m.router"]), ids, wts, top, "softmax_chosen")
        idx, score = plain.router_choice(h, w["m.router"], top)
        assert np.array_equal(ids.cpu().numpy(), idx)
        assert np.abs(f64(wts) - score).max() < 2e-6
        assert np.abs(f64(wts).sum(axis=1) - 1.0).max() < 1e-5
        gate_up = np.concatenate([np.concatenate([w[f"m.e{e}.gate"], w[f"m.e{e}.up"]]) for e in range(E)])
        down = np.concatenate([w[f"m.e{e}.down"] for e in range(E)])
        y = torch.full((M, W), 5.0, device="cuda")
        ops.moe_experts_gated(dev(h, DT[dtype]), ids, wts, dev(gate_up, DT[dtype]), dev(down, DT[dtype]), y, E, "clamped", limit)
        want = plain.moe(h, w, "m", dict(router=dict(experts=E, top=top), expert=dict(limit=limit)))
        tol = 2e-5 if dtype == "float32" else 2e-2
        assert np.abs(f64(y) - want).max() < tol * max(1.0, np.abs(want).max()), (M, E)


def test_equal_logits_go_to_the_lower_index(ops):
    h = np.zeros((2, 8))
    h[1, 0] = 1.0
    router = np.zeros((70, 8))
    router[[5, 66, 69], 0] = 2.0
    ids = torch.empty(2, 3, device="cuda", dtype=torch.int32)
    wts = torch.empty(2, 3, device="cuda")
    ops.moe_route(dev(h), dev(router), ids, wts, 3, "softmax_chosen")
    assert ids.cpu().numpy().tolist() == [[0, 1, 2], [5, 66, 69]]
    assert np.allclose(f64(wts), 1.0 / 3.0)


# --------------------------------------------------------------------------------------- the engine
REQUEST_LENGTHS = {"a": 97, "b": 45, "c": 130, "d": 33, "e": 71, "f": 58}
PROMPT_LENGTHS = {"a": 60, "b": 12, "c": 101, "d": 30, "e": 2, "f": 41}
_made = {}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    def get(name):
        if name not in _made:
            config = nm.CONFIGS[name]
            weights = nm.draw_weights(config, seed=len(name) * 13 + 2)
            path = nm.write_folder(str(tmp_path_factory.mktemp("nazorax_" + name)), config, 0, weights)
            requests = {r: random_tokens(n, config["vocab"], 17 + i) for i, (r, n) in enumerate(REQUEST_LENGTHS.items())}
            w = nm.as_float64(weights)
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
@pytest.mark.parametrize("name,page_size", [("looped", 8), ("odd", 4), ("wide", 16)])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_engine_matches_plain(folders, name, page_size, dtype, mode):
    folder, requests, want, _ = folders(name)
    trace = make_trace(mode, requests)
    n_tok = traces.max_pages(trace, page_size) * page_size      # the tightest pool: pages are handed out again
    engine = build_engine(folder, dtype, n_tok, page_size)
    got = replay(engine, trace)
    assert not engine.cache.live_requests()
    ok, seen = within(got, want, dtype)
    assert ok, (name, mode, dtype, seen)


@pytest.mark.parametrize("name", ["looped", "odd"])
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


def test_pages_used_again_hold_nothing_of_their_last_owner(folders):
    """One request at a time in the smallest pool that holds it: the second gets the pages the first gave back."""
    folder, requests, want, _ = folders("looped")
    engine = build_engine(folder, "float32", 144, page_size=8, max_requests=1)
    for r in ("c", "b", "c"):
        got = replay(engine, traces.portions({r: requests[r]}))
        w, where = worst(got, {r: want[r]})
        assert w < TOL["float32"], (r, w, where)


def test_long_decoding_past_every_window(folders):
    """A prompt of 50 tokens in portions of 32, then 250 tokens one by one: the decoded tokens leave the windows of 21 and
    40 far behind (pages of 8 go back behind them) while the latent layers keep every token."""
    from tinyinfer_amd.engine import StepEntry
    folder, _, _, w = folders("looped")
    config = nm.CONFIGS["looped"]
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


def test_a_token_far_back_reaches_the_last_position_through_the_latent_layers_only(folders):
    """Changing token 3 of 120 moves the last position's logits (the latent layers see everything); in a model cut down to
    its window layers it does not."""
    from tinyinfer_amd.engine import StepEntry
    folder, requests, _, w = folders("looped")
    config = nm.CONFIGS["looped"]
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
    folder, requests, _, w = folders("looped")
    config = nm.CONFIGS["looped"]
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


def test_graphs_replay_the_matrix_core_kernels(folders):
    """bfloat16 at sizes the matrix-core kernels of both mixers serve: decoding from captured graphs gives the tokens that
    decoding step by step gives."""
    import tinyinfer_amd as ti
    folder, requests, _, _ = folders("wide")
    prompts = [requests["b"][:37], requests["d"][:5], requests["e"][:50]]
    outs = []
    for use_graph in (False, True):
        llm = ti.LLM(folder, dtype="bfloat16", max_seq=128, max_requests=3, chunk_size=32, max_batched_tokens=64, use_graph=use_graph)
        outs.append(llm.generate(prompts, max_new_tokens=20, temperature=0.0))
    assert outs[0] == outs[1]


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


def test_command_line_generates_from_a_nazorax_folder(folders):
    """bin/tinyinfer picks the model by config.json: token ids in, the plain model's greedy tokens out; with --cuda-graph too."""
    import os
    import subprocess
    import sys
    folder, requests, _, w = folders("odd")
    config = nm.CONFIGS["odd"]
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
    for name in ("looped", "wide"):
        engine = Engine.from_config(nm.CONFIGS[name], seed=3, dtype="bfloat16", page_size=16, max_tokens=256, max_requests=2, max_seq=256)
        toks = random_tokens(70, nm.CONFIGS[name]["vocab"], 1)
        a = engine.step([StepEntry("x", toks, [69])]).cpu().numpy()
        engine.release("x")
        assert engine.step([StepEntry("y", toks[:69], [])]) is None
        b = engine.step([StepEntry("y", toks[69:], [0])]).cpu().numpy()
        assert np.isfinite(a).all() and a.std() > 0
        assert np.abs(a - b).max() < 0.08 * max(1e-6, np.abs(a).max())


def test_trace_replay_program(folders, tmp_path):
    """The replay program on a Nazorax folder: it picks the model by config.json and writes the logits the engine gives."""
    import os
    import subprocess
    import sys
    folder, requests, want, _ = folders("odd")
    some = {r: requests[r] for r in ("b", "d", "f")}
    trace = traces.mixed(some, PROMPT_LENGTHS, live=2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", str(traces.max_tokens(trace))], input=traces.to_jsonl(trace), text=True,
                          capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    V = nm.CONFIGS["odd"]["vocab"]
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
