"""Operator selftest: every kernel against a plain float64 computation on the CPU, in the
manner of the reference's `QWEN_SELFTEST=1` (/root/reference/src/selftest.cpp:463-473; its
cases and tolerances: 33-72 product, 74-100 RMSNorm, 102-134 rotation, 136-390 per-head
norm + rotation + cache + attention, 392-459 products of the model's shapes with timings).

    TINY_SELFTEST=1 bin/tinyinfer          or          python -m tinyinfer_amd.selftest

The exit code is the number of failed cases.  The cases keep the reference's sizes where the
reference names them; operands are drawn from a seeded generator, rounded to bfloat16 where
the kernels take bfloat16, and the CPU side computes in float64 from those same values.
"""
from __future__ import annotations

import math
import sys
import time

import numpy as np
import torch


def _say(name: str, err: float, tol: float, extra: str = "") -> int:
    ok = err < tol and math.isfinite(err)
    print(f"[selftest] {name:46s} max err {err:.3e}  (< {tol:.1e})  {'ok' if ok else 'FAIL'}{extra}", flush=True)
    return 0 if ok else 1


def _dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def _f64(t) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def _bf16(a: np.ndarray) -> np.ndarray:
    """Round to bfloat16 (nearest even) and come back as float64."""
    return torch.as_tensor(a, dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()


class _View:
    def __init__(self, table):
        self.table = table


class _Ctx:
    """What the attention dispatch reads of a step: rows of single tokens, or one portion."""

    def __init__(self, positions, one_portion: bool):
        M = len(positions)
        self.M = M
        self.positions = _dev(np.asarray(positions, dtype=np.int32))
        self.slots = _dev(np.zeros(M, dtype=np.int32))
        self.decode_only = not one_portion
        self.decode_rows, self.n_decode_rows = None, 0
        self.n_tiles = -(-M // 128) if one_portion else 0
        self.tiles = _dev(np.array([[0, 128 * i] for i in range(self.n_tiles)], dtype=np.int32)) if one_portion else None
        self.n_tiles_small = -(-M // 64) if one_portion else 0     # from the most keys to the fewest
        self.tiles_small = _dev(np.array([[0, 64 * i] for i in reversed(range(self.n_tiles_small))],
                                         dtype=np.int32)) if one_portion else None
        self.entry_meta = _dev(np.array([[0, M, positions[0], 0]], dtype=np.int32))
        self.max_context = self.split_context = int(max(positions)) + 1

    def buf(self, name, shape, dtype):
        return torch.empty(tuple(shape), dtype=dtype, device="cuda")


# ------------------------------------------------------------------ the cases
def case_linear(ops, rng) -> int:
    fails = 0
    M, N, K = 5, 261, 1024                       # the reference's case: N odd, bounds of the tiles
    a, w = _bf16(rng.uniform(-1, 1, (M, K))), _bf16(rng.uniform(-1, 1, (N, K)))
    want = a @ w.T
    for dtype in (torch.bfloat16, torch.float32):
        out = torch.empty(M, N, device="cuda")
        ops.linear(_dev(a, dtype), _dev(w, dtype), out, "store")
        fails += _say(f"product {M}x{N}x{K} {str(dtype)[6:]}", float(np.abs(_f64(out) - want).max()), 2e-5 * K)
    # all epilogues at a size that is no multiple of anything, many rows (the tiled kernels)
    M, N, K = 203, 130, 192
    a, w = _bf16(rng.uniform(-1, 1, (M, K))), _bf16(rng.uniform(-1, 1, (N, K)))
    base = rng.normal(size=(M, N)).astype(np.float32)
    want = a @ w.T
    out = _dev(base.copy())
    ops.linear(_dev(a, torch.bfloat16), _dev(w, torch.bfloat16), out, "add")
    fails += _say("product + residual add", float(np.abs(_f64(out) - (want + base)).max()), 2e-5 * K + 1e-5)
    F = N // 2
    g, u = want[:, :F], want[:, F:]
    out = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
    ops.linear(_dev(a, torch.bfloat16), _dev(w, torch.bfloat16), out, "swiglu")
    swi = g / (1 + np.exp(-g)) * u
    fails += _say("product + SwiGLU (bfloat16 out)", float(np.abs(_f64(out) - swi).max()), 0.005 * np.abs(swi).max() + 1e-3)
    # few rows times a long K (the token rows go through LDS in pieces; with a long K under few weight
    # rows the sums of several workgroups are left to whatever reads the residual next)
    for M, N, K in ((7, 2100, 5120), (16, 2064, 17408)):
        a, w = _bf16(rng.uniform(-1, 1, (M, K))), _bf16(rng.uniform(-1, 1, (N, K)))
        base = rng.normal(size=(M, N)).astype(np.float32)
        out = _dev(base.copy())
        ops.linear(_dev(a, torch.bfloat16), _dev(w, torch.bfloat16), out, "add", may_defer=True)
        ops.flush()
        fails += _say(f"product {M}x{N}x{K} + residual add (K in pieces)", float(np.abs(_f64(out) - (a @ w.T + base)).max()),
                      2e-5 * K)
    return fails


def case_model_shapes(ops, rng) -> int:
    """The projections of a 0.6B layer at two rows, with timings (reference: printed only)."""
    fails = 0
    for N, K in ((4096, 1024), (2048, 1024), (1024, 1024), (1024, 3072), (2048, 3072)):
        a, w = _bf16(rng.uniform(-1, 1, (2, K))), _bf16(rng.uniform(-1, 1, (N, K)) * 0.05)
        ad, wd = _dev(a, torch.bfloat16), _dev(w, torch.bfloat16)
        out = torch.empty(2, N, device="cuda")
        ops.linear(ad, wd, out, "store")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(100):
            ops.linear(ad, wd, out, "store")
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) / 100 * 1e6
        fails += _say(f"product 2x{N}x{K} (a layer's shape)", float(np.abs(_f64(out) - a @ w.T).max()), 0.02,
                      f"  {us:6.1f} us  {N * K * 2 / us / 1e3:6.0f} GB/s")
    return fails


def case_rmsnorm(ops, rng) -> int:
    rows, n, eps = 3, 1024, 1e-6
    x, w = rng.uniform(-1, 1, (rows, n)).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    xd = x.astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(-1, keepdims=True) + eps) * w
    out = torch.empty(rows, n, device="cuda")
    ops.rmsnorm(_dev(x), _dev(w), eps, out)
    fails = _say("RMSNorm 3x1024", float(np.abs(_f64(out) - want).max()), 1e-4)
    # rows wider than 4,096 take a workgroup each
    rows, n = 5, 5120
    x, w = rng.uniform(-1, 1, (rows, n)).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    xd = x.astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(-1, keepdims=True) + eps) * w
    out = torch.empty(rows, n, device="cuda")
    ops.rmsnorm(_dev(x), _dev(w), eps, out)
    fails += _say("RMSNorm 5x5120", float(np.abs(_f64(out) - want).max()), 1e-4)
    return fails


def _rotate(x, positions, theta):
    """x [M, heads, hd] float64; pairs (k, k + hd/2), angle pos * theta^(-2k/hd)."""
    hd = x.shape[-1]
    half = hd // 2
    ang = np.asarray(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * np.arange(half) / hd)[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate([lo * c - hi * s, lo * s + hi * c], axis=-1)


def case_rope(ops, rng) -> int:
    rows, heads, hd, theta = 2, 4, 128, 1e6
    x = rng.uniform(-1, 1, (rows, heads, hd)).astype(np.float32)
    pos = [0, 5]
    inv = (theta ** (-2.0 * np.arange(hd // 2) / hd)).astype(np.float32)
    xd = _dev(x)
    ops.rope_neox(xd, _dev(np.asarray(pos, dtype=np.int32)), _dev(inv))
    return _say("rotation 2x4x128, positions 0 and 5", float(np.abs(_f64(xd) - _rotate(x.astype(np.float64), pos, theta)).max()), 1e-4)


def case_attention(ops, rng, nh, nkv, hd, T, dtype, eps=1e-6, theta=1e6, P=16) -> int:
    """Per-head norm, rotation, cache write and causal attention of T tokens of one request: as one
    portion, and as T steps of one token; against float64 from the rounded cache values."""
    name = f"norm+rotation+cache+attention hd={hd} {nh}/{nkv} heads {str(dtype)[6:]}"
    width = (nh + 2 * nkv) * hd
    qkv = rng.uniform(-1, 1, (T, width)).astype(np.float32)
    q_w, k_w = rng.uniform(0.5, 1.5, hd).astype(np.float32), rng.uniform(0.5, 1.5, hd).astype(np.float32)
    inv = (theta ** (-2.0 * np.arange(hd // 2) / hd)).astype(np.float32)

    def heads(a, n):
        return a.reshape(T, n, hd).astype(np.float64)

    def norm(a, w):
        return a / np.sqrt((a * a).mean(-1, keepdims=True) + eps) * w
    pos = list(range(T))
    rnd = _bf16 if dtype == torch.bfloat16 else (lambda z: z)
    q = rnd(_rotate(norm(heads(qkv[:, :nh * hd], nh), q_w), pos, theta))
    k = rnd(_rotate(norm(heads(qkv[:, nh * hd:(nh + nkv) * hd], nkv), k_w), pos, theta))
    v = rnd(heads(qkv[:, (nh + nkv) * hd:], nkv))
    want = np.zeros((T, nh, hd))
    for h in range(nh):
        s = q[:, h] @ k[:, h // (nh // nkv)].T / math.sqrt(hd)
        s[np.triu_indices(T, 1)] = -np.inf
        p = np.exp(s - s.max(-1, keepdims=True))
        want[:, h] = (p / p.sum(-1, keepdims=True)) @ v[:, h // (nh // nkv)]
    want = want.reshape(T, nh * hd)
    n_pages = -(-T // P) + 1
    table = _dev(np.arange(n_pages, dtype=np.int32)[::-1].copy()[None, :])     # pages in descending order
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    fails = 0
    for mode in ("one portion", "token by token"):
        pool = torch.zeros(n_pages, 2, nkv, P, hd, device="cuda", dtype=dtype)
        got = torch.empty(T, nh * hd, device="cuda", dtype=dtype)
        steps = [pos] if mode == "one portion" else [[p] for p in pos]
        for rows in steps:
            ctx = _Ctx(rows, one_portion=(mode == "one portion"))
            qd = torch.empty(len(rows), nh * hd, device="cuda", dtype=dtype)
            ops.qk_norm_rope_kv_write(_dev(qkv[rows]), _dev(q_w), _dev(k_w), eps, _dev(inv), ctx.positions, ctx.slots,
                                      _View(table), pool, qd, nh, nkv, hd)
            out = torch.empty_like(qd)
            ops.attention(ctx, _View(table), qd, pool, out, nh, nkv, hd, 1.0 / math.sqrt(hd), None)
            got[rows[0]:rows[-1] + 1] = out
        fails += _say(f"{name}, {mode}", float(np.abs(_f64(got) - want).max()), tol)
    return fails


def case_embed_argmax_sample(ops, rng) -> int:
    fails = 0
    V, H = 1000, 96
    E = _bf16(rng.normal(size=(V, H)))
    toks = np.array([5, 0, 999, 5], dtype=np.int32)
    x = torch.empty(4, H, device="cuda")
    ops.embed(_dev(E, torch.bfloat16), _dev(toks), x)
    fails += _say("embedding rows", float(np.abs(_f64(x) - E[toks]).max()), 1e-12)
    logits = rng.normal(size=(3, 151936)).astype(np.float32)
    logits[1, 77] = logits[1, 4000] = 9.0                        # a tie: the lowest index wins
    out = torch.empty(3, dtype=torch.int32, device="cuda")
    ops.argmax(_dev(logits), out)
    fails += _say("argmax, ties to the lowest index", float(np.abs(out.cpu().numpy() - logits.argmax(-1)).max()), 0.5)
    # temperature sampling: the token is where the inverse CDF of softmax(logits / T) crosses u
    small = rng.normal(size=(2, 50)).astype(np.float32) * 3
    T, u = 0.7, np.array([0.25, 0.9], dtype=np.float32)
    z = small.astype(np.float64) / T
    p = np.exp(z - z.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    cdf = np.cumsum(p, -1)
    got = torch.empty(2, dtype=torch.int32, device="cuda")
    ops.sample(_dev(small), _dev(np.full(2, T, dtype=np.float32)), _dev(np.full(2, 50, dtype=np.int32)),
               _dev(np.ones(2, dtype=np.float32)), _dev(u), got)
    tok = got.cpu().numpy()
    # u must fall into the drawn token's interval of the cumulative distribution
    miss = max(max(cdf[i, tok[i]] - p[i, tok[i]] - u[i], u[i] - cdf[i, tok[i]], 0.0) for i in range(2))
    fails += _say("temperature sampling, inverse CDF", float(miss), 1e-4)
    return fails


def case_head_bandwidth(ops, rng) -> int:
    """One row through an output matrix of the real vocabulary (reference: timing only)."""
    N, K = 151936, 1024
    w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.bfloat16)
    a = torch.randn(1, K, device="cuda").to(torch.bfloat16)
    out = torch.empty(1, N, device="cuda")
    ops.linear(a, w, out, "store")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        ops.linear(a, w, out, "store")
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) / 20 * 1e6
    want = _f64(a) @ _f64(w[:64]).T
    return _say("product 1x151936x1024 (the output matrix)", float(np.abs(_f64(out[:, :64]) - want).max()), 0.02,
                f"  {us:6.1f} us  {N * K * 2 / us / 1e3:6.0f} GB/s")


def case_pointwise(ops, rng) -> int:
    """The element-wise kernels of parallel layers: sinusoidal positions, xIELU, the scaled sum into the residual."""
    fails = 0
    H, pos = 48, np.array([0, 7, 640, 3000], dtype=np.int32)
    inv = np.array([10000.0 ** (-2.0 * i / H) for i in range(H // 2)], dtype=np.float32)
    x0 = rng.normal(size=(len(pos), H)).astype(np.float32)
    x = _dev(x0)
    ops.add_sinusoid(x, _dev(pos), _dev(inv))
    angle = pos[:, None].astype(np.float64) * inv[None, :].astype(np.float64)
    want = x0.astype(np.float64)
    want[:, 0::2] += np.sin(angle)
    want[:, 1::2] += np.cos(angle)
    fails += _say("sinusoidal positions added (32-bit angles)", float(np.abs(_f64(x) - want).max()), 5e-4)
    z = (rng.normal(size=(16, 64)) * 3).astype(np.float32)
    u, v = 0.4, -0.6
    sp = lambda t: math.log1p(math.exp(t))      # noqa: E731
    zz = z.astype(np.float64)
    want = np.where(zz > 0, sp(u) * zz * zz + 0.5 * zz, (0.5 + sp(v)) * (np.expm1(np.minimum(zz, 0)) - np.minimum(zz, 0)) + 0.5 * zz)
    for dt, tol in ((torch.float32, 1e-4), (torch.bfloat16, 0.2)):
        out = torch.empty(16, 64, device="cuda", dtype=dt)
        ops.xielu(_dev(z), _dev(np.array([u, v], dtype=np.float32)), out)
        fails += _say(f"xIELU 16x64 -> {str(dt).split('.')[-1]}", float(np.abs(_f64(out) - want).max()), tol)
    a, b = rng.normal(size=(16, 48)).astype(np.float32), rng.normal(size=(16, 48)).astype(np.float32)
    sa, sb = rng.normal(size=48).astype(np.float32), rng.normal(size=48).astype(np.float32)
    x0 = rng.normal(size=(16, 48)).astype(np.float32)
    x = _dev(x0)
    ops.scaled_add(x, _dev(a), _dev(sa), _dev(b), _dev(sb))
    want = x0.astype(np.float64) + a.astype(np.float64) * sa + b.astype(np.float64) * sb
    fails += _say("scaled sum of two branches into the residual", float(np.abs(_f64(x) - want).max()), 1e-5)
    return fails


def case_capped_attention(ops, rng, nh, nkv, dk, dv, T, dtype) -> int:
    """q/k/v split with a query temperature into pages (K [kv][P][dk] | V [kv][dv][P]), then soft-capped attention of every row."""
    P, cap, coef, every, scale = 16, 5.0, 0.3, 4, 1.0 / math.sqrt(dk)
    q, k, v = rng.normal(size=(T, nh, dk)) * 1.5, rng.normal(size=(T, nkv, dk)), rng.normal(size=(T, nkv, dv))
    qkv = np.concatenate([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], axis=1).astype(np.float32)
    pages = -(-T // P)
    table = rng.permutation(pages + 2)[:pages].astype(np.int32)[None, :]
    pool = torch.zeros(pages + 2, nkv, P, dk + dv, device="cuda", dtype=dtype)
    q_out = torch.empty(T, nh * dk, device="cuda", dtype=dtype)
    pos, slots = _dev(np.arange(T, dtype=np.int32)), _dev(np.zeros(T, dtype=np.int32))
    ops.qkv_split_write(_dev(qkv), pos, slots, _dev(table), pool, q_out, nh, nkv, dk, dv, coef, every)
    out = torch.empty(T, nh * dv, device="cuda", dtype=dtype)
    ops.attention_capped(q_out, pool, _dev(table), pos, slots, out, nh, nkv, dk, dv, scale, cap)
    rnd = _bf16 if dtype == torch.bfloat16 else (lambda t: np.asarray(t, dtype=np.float32).astype(np.float64))
    temp = np.array([1 + coef * math.log((p + 1) // every + 1) for p in range(T)])
    qt, kr, vr = _f64(q_out).reshape(T, nh, dk), rnd(k), rnd(v)
    err_q = float(np.abs(qt - rnd(q * temp[:, None, None])).max() / np.abs(qt).max())
    want = np.zeros((T, nh, dv))
    for i in range(T):
        for h in range(nh):
            g = h // (nh // nkv)
            s = cap * np.tanh((kr[: i + 1, g] @ qt[i, h]) * scale / cap)
            p = np.exp(s - s.max())
            want[i, h] = (p / p.sum()) @ vr[: i + 1, g]
    name = f"capped attention {nh}/{nkv} heads, {dk}/{dv}, {T} tokens, {str(dtype).split('.')[-1]}"
    fails = _say(name + ": q", err_q, 1e-5 if dtype == torch.float32 else 1e-2)
    return fails + _say(name, float(np.abs(_f64(out).reshape(T, nh, dv) - want).max()), 1e-4 if dtype == torch.float32 else 2e-2)


def case_mlstm(ops, rng, heads, dk, dv, lengths, chunk) -> int:
    """The mLSTM scan over several requests (whole, and cut into chunks that run side by side), then the gated head norm."""
    cap, N = 6.0, heads * (2 * dk + 2 * dv + 2)
    cq, ck, cv, cg = 0, heads * dk, 2 * heads * dk, 2 * heads * dk + heads * dv
    ci, cf = cg + heads * dv, cg + heads * dv + heads
    M = sum(lengths)
    proj = rng.normal(size=(M, N)).astype(np.float32)
    bi, bf = rng.normal(size=heads).astype(np.float32), (rng.normal(size=heads) + 2).astype(np.float32)
    entries, chunks, spans, row = [], [], [], 0
    for e, n_tok in enumerate(lengths):
        entries.append([row, n_tok, 0, e])
        n = -(-n_tok // chunk)
        spans.append([len(chunks), n])
        chunks += [[e, row + j * chunk, min(chunk, n_tok - j * chunk), (j == 0) | 2 * (j == n - 1)] for j in range(n)]
        row += n_tok
    p = proj.astype(np.float64)
    want = np.zeros((M, heads, dv))
    for row0, n_tok, _, _ in entries:
        for h in range(heads):
            S, n, m = np.zeros((dk, dv)), np.zeros(dk), 0.0
            for t in range(row0, row0 + n_tok):
                q, k, v = p[t, cq + h * dk: cq + (h + 1) * dk] * float(np.float32(dk ** -0.5)), p[t, ck + h * dk: ck + (h + 1) * dk], p[t, cv + h * dv: cv + (h + 1) * dv]
                ig = cap * math.tanh((p[t, ci + h] + bi[h]) / cap)
                fz = cap * math.tanh((p[t, cf + h] + bf[h]) / cap)
                fg = min(fz, 0.0) - math.log1p(math.exp(-abs(fz)))
                m_new = max(fg + m, ig)
                S = math.exp(fg + m - m_new) * S + math.exp(ig - m_new) * np.outer(k, v)
                n = math.exp(fg + m - m_new) * n + math.exp(ig - m_new) * k
                m = m_new
                want[t, h] = (S.T @ q) / (max(abs(float(n @ q)), math.exp(-m)) + 1e-6)
    fails = 0
    o = None
    for how in ("token by token", "in chunks"):
        state = torch.zeros(len(lengths), heads, dk * dv + dk + 1, device="cuda")
        o = torch.empty(M, heads * dv, device="cuda")
        more = {} if how == "token by token" else dict(chunks=_dev(np.array(chunks, dtype=np.int32)), spans=_dev(np.array(spans, dtype=np.int32)))
        ops.mlstm_scan(_dev(proj), _dev(bi), _dev(bf), state, _dev(np.array(entries, dtype=np.int32)), o, heads, dk, dv, cap, dk ** -0.5,
                       (cq, ck, cv, ci, cf), **more)
        err = float(np.abs(_f64(o).reshape(M, heads, dv) - want).max() / max(1.0, np.abs(want).max()))
        fails += _say(f"mLSTM scan {heads} heads {dk}x{dv}, {lengths} tokens, {how}", err, 3e-4)
    w = rng.normal(size=heads * dv).astype(np.float32)
    out = torch.empty(M, heads * dv, device="cuda")
    ops.gated_head_norm(o, _dev(proj), cg, _dev(w), 1e-5, out, heads, dv)
    oo = _f64(o).reshape(M, heads, dv)
    normed = (oo / np.sqrt((oo * oo).mean(-1, keepdims=True) + 1e-5)).reshape(M, -1) * w / (1 + np.exp(-p[:, cg: cg + heads * dv]))
    return fails + _say("gated head norm", float(np.abs(_f64(out) - normed).max()), 1e-4)


def case_norm_residual_and_experts(ops, rng) -> int:
    """The norm onto the residual (with rows gathered on the way and a rounded copy), the router and the experts, row-wise
    in 32-bit and bfloat16 and grouped on the matrix cores."""
    fails = 0
    M, H = 6, 200
    x0, y, g = rng.normal(size=(M, H)), rng.normal(size=(9, H)) * 2, 1 + 0.2 * rng.normal(size=H)
    gather = rng.integers(0, 9, size=(M, 2)).astype(np.int32)
    x, copy = _dev(x0, torch.float32), torch.empty(M, H, device="cuda", dtype=torch.bfloat16)
    ops.norm_residual(x, _dev(y, torch.float32), _dev(g, torch.float32), 1e-5, True, _dev(gather), copy)
    yy = y[gather[:, 0]] + y[gather[:, 1]]
    want = x0 + yy / np.sqrt((yy * yy).mean(-1, keepdims=True) + 1e-5) * g
    fails += _say("norm onto the residual, rows gathered", float(np.abs(_f64(x) - want).max()), 5e-6)
    fails += _say("  its rounded copy", float(np.abs(_f64(copy) - _bf16(_f64(x))).max()), 1e-12)
    for dtype, M, W, E, top, F, tol in ((torch.float32, 7, 96, 6, 2, 80, 3e-5), (torch.bfloat16, 5, 64, 4, 3, 96, 2e-2),
                                        (torch.bfloat16, 400, 128, 9, 2, 160, 2e-2)):
        h = _bf16(rng.normal(size=(M, W)))
        router = (rng.normal(size=(E, W)) * 2 / math.sqrt(W)).astype(np.float32)
        up, down = _bf16(rng.normal(size=(E, F, W)) / math.sqrt(W)), _bf16(rng.normal(size=(E, W, F)) / math.sqrt(F))
        ids, wts = torch.empty(M, top, device="cuda", dtype=torch.int32), torch.empty(M, top, device="cuda")
        ops.moe_route(_dev(h, dtype), _dev(router), ids, wts, top)
        score = 1 / (1 + np.exp(-(h @ router.astype(np.float64).T)))
        order = np.argsort(-score, axis=1, kind="stable")[:, :top]
        name = f"experts {top} of {E}, {M} tokens, {W} -> {F}, {str(dtype).split('.')[-1]}"
        fails += _say(name + ": choice", float((ids.cpu().numpy() != order).sum()), 0.5)
        out = torch.empty(M, W, device="cuda")
        ops.moe_experts(_dev(h, dtype), ids, wts, _dev(up.reshape(E * F, W), dtype), _dev(down.reshape(E * W, F), dtype), out, E)
        want = np.zeros((M, W))
        for m in range(M):
            for e in order[m]:
                want[m] += (np.maximum((score[m, e] * h[m]) @ up[e].T, 0) ** 2) @ down[e].T
        fails += _say(name, float(np.abs(_f64(out) - want).max() / max(1.0, np.abs(want).max())), tol)
    return fails


def case_diff_attention(ops, rng, nh, nkv, dk, dv, T, block, taps, rot, dtype, P=16) -> int:
    """Short convolution, per-map norm, partial rotation and cache write in one kernel, then differential attention of every
    row (row-wise, and for bfloat16 sizes the matrix-core kernels take: as tiles of a portion and as single tokens)."""
    eps, lam, out_scale, scale = 1e-5, 0.7, 0.5, 1 / math.sqrt(dk)
    C = nh * 2 * dk + nkv * (2 * dk + dv)
    u = rng.normal(size=(T, C)).astype(np.float32)
    tp = rng.normal(size=(C, taps)).astype(np.float32)
    qw, kw = (1 + 0.2 * rng.normal(size=dk)).astype(np.float32), (1 + 0.2 * rng.normal(size=dk)).astype(np.float32)
    freq = np.array([100.0 ** (-2.0 * i / max(rot, 1)) for i in range(rot // 2)], dtype=np.float32)
    n_pages = -(-T // P)
    table = rng.permutation(n_pages).astype(np.int32)[None, :]
    pool = torch.zeros(n_pages, nkv, P, 2 * dk + dv, device="cuda", dtype=dtype)
    q_out = torch.empty(T, nh * 2 * dk, device="cuda", dtype=dtype)
    pos, slots = _dev(np.arange(T, dtype=np.int32)), _dev(np.zeros(T, dtype=np.int32))
    state = torch.zeros(1, taps - 1, C, device="cuda")
    entries = _dev(np.array([[0, T, 0, 0]], dtype=np.int32))
    ops.diff_qk_prep(_dev(u), _dev(qw), _dev(kw), _dev(freq) if rot else None, None, pos, slots, _dev(table), pool, q_out, eps, nh, nkv,
                     dk, dv, rot, 1.0, taps=_dev(tp), state=state, entries=entries)
    pad = np.concatenate([np.zeros((taps - 1, C)), u.astype(np.float64)])
    mixed = sum(pad[j:j + T] * tp[:, j].astype(np.float64) for j in range(taps))
    q = mixed[:, :nh * 2 * dk].reshape(T, nh, 2, dk)
    k = mixed[:, nh * 2 * dk: nh * 2 * dk + nkv * 2 * dk].reshape(T, nkv, 2, dk)
    v = mixed[:, nh * 2 * dk + nkv * 2 * dk:].reshape(T, nkv, dv)

    def prepare(z, w):
        z = z / np.sqrt((z * z).mean(-1, keepdims=True) + eps) * w
        out = z.copy()
        for t in range(T):
            a = np.float64(np.float32(t) * freq)
            out[t, ..., :rot // 2] = z[t, ..., :rot // 2] * np.cos(a) - z[t, ..., rot // 2:rot] * np.sin(a)
            out[t, ..., rot // 2:rot] = z[t, ..., rot // 2:rot] * np.cos(a) + z[t, ..., :rot // 2] * np.sin(a)
        return out
    rnd = _bf16 if dtype == torch.bfloat16 else (lambda t: t)
    qn, kn, vn = rnd(prepare(q, qw)), rnd(prepare(k, kw)), rnd(v)
    name = f"differential attention {nh}/{nkv} heads, {dk}/{dv}, {T} tokens, blocks of {block}, {taps} taps, {str(dtype).split('.')[-1]}"
    fails = _say(name + ": q", float(np.abs(_f64(q_out).reshape(T, nh, 2, dk) - qn).max() / np.abs(qn).max()), 3e-5 if dtype == torch.float32 else 1e-2)
    fails += _say(name + ": state left", float(np.abs(_f64(state)[0] - u[T - taps + 1:]).max()), 1e-12)
    want = np.zeros((T, nh, dv))
    for i in range(T):
        lo = i // block * block
        for h in range(nh):
            g = h // (nh // nkv)
            a = []
            for mp in range(2):
                s = (kn[lo: i + 1, g, mp] @ qn[i, h, mp]) * scale
                p = np.exp(s - s.max())
                a.append((p / p.sum()) @ vn[lo: i + 1, g])
            o = a[0] - lam * a[1]
            want[i, h] = o / math.sqrt((o * o).mean() + eps) * out_scale
    want = want.reshape(T, -1)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    out = torch.empty(T, nh * dv, device="cuda", dtype=dtype)
    args = (q_out, pool, _dev(table), pos, slots)
    ops.diff_attention(*args, out, nh, nkv, dk, dv, scale, lam, eps, out_scale, block=block)
    fails += _say(name, float(np.abs(_f64(out) - want).max()), tol)
    if dtype == torch.bfloat16 and dk in (32, 64, 128) and dv in (32, 64, 128):
        tiles = _dev(np.array([[0, r, min(64, T - r)] for r in range(0, T, 64)], dtype=np.int32))
        ops.diff_attention(*args, out, nh, nkv, dk, dv, scale, lam, eps, out_scale, block=block, tiles=tiles, entries=entries)
        fails += _say(name + ", tiles on the matrix cores", float(np.abs(_f64(out) - want).max()), tol)
        ops.diff_attention(*args, out, nh, nkv, dk, dv, scale, lam, eps, out_scale, block=block, all_rows=True)
        fails += _say(name + ", single tokens on the matrix cores", float(np.abs(_f64(out) - want).max()), tol)
    return fails


def case_streams_gates_and_decay(ops, rng) -> int:
    """The layer norm of a weighted sum of streams, the write into the streams, attention with a sink and a gate over pages,
    and linear attention with a fixed decay whole and in chunks, each against a host computation."""
    fails = 0

    def D(a):      # 64-bit host arrays go to the device as float32, integer lists as they are
        a = np.asarray(a)
        return _dev(a.astype(np.float32) if a.dtype == np.float64 else a)

    S, M, W = 3, 21, 70
    xs, coef, back = rng.normal(size=(S, M, W)), rng.normal(0.5, 0.4, size=S), rng.normal(1.0, 0.4, size=S)
    mix, g, y = np.eye(S) + rng.normal(0, 0.3, size=(S, S)), rng.normal(1.0, 0.2, size=W), rng.normal(size=(M, W))
    f32 = lambda a: np.asarray(a, dtype=np.float32).astype(np.float64)
    u = np.einsum("s,smw->mw", f32(coef), f32(xs))
    d = u - u.mean(-1, keepdims=True)
    want = d / np.sqrt((d * d).mean(-1, keepdims=True) + 1e-6) * f32(g)
    streams, out = D(xs), torch.empty(M, W, device="cuda")
    ops.layernorm_mixed(streams, D(coef), D(g), 1e-6, out)
    fails += _say("layer norm of a weighted sum of 3 streams", float(np.abs(_f64(out) - want).max()), 5e-5)
    ops.hyper_write(streams, D(mix), D(back), D(y))
    want = np.einsum("st,smw->tmw", f32(mix), f32(xs)) + f32(back)[:, None, None] * f32(y)[None]
    fails += _say("write into 3 streams", float(np.abs(_f64(streams) - want).max()), 2e-5)
    # attention with a sink and a gate a head, keys 24 and values 40, pages of 8
    T, nh, nkv, dk, dv, P = 70, 4, 2, 24, 40, 8
    nq, nk, nv = nh * dk, nkv * dk, nkv * dv
    proj = rng.normal(size=(T, nq + nk + nv + nh))
    sink = rng.normal(0.5, 1.0, size=nh)
    n_pages = -(-T // P)
    table = rng.permutation(n_pages + 2)[:n_pages].astype(np.int32)[None, :]
    pos, slots = np.arange(T, dtype=np.int32), np.zeros(T, dtype=np.int32)
    for dtype, tol in ((torch.float32, 5e-5), (torch.bfloat16, 3e-2)):
        pool = torch.zeros(n_pages + 2, nkv, P, dk + dv, device="cuda", dtype=dtype)
        q_out = torch.empty(T, nq, device="cuda", dtype=dtype)
        args = (D(pos), D(slots), D(table))
        ops.gated_qkv_prep(D(proj), None, None, None, None, *args, pool, q_out, nh, nkv, dk, dv, (0, nq, nq + nk))
        p32 = f32(proj)
        rnd = _bf16 if dtype == torch.bfloat16 else (lambda a: a)
        q, k = rnd(p32[:, :nq]).reshape(T, nh, dk), rnd(p32[:, nq:nq + nk]).reshape(T, nkv, dk)
        v = rnd(p32[:, nq + nk:nq + nk + nv]).reshape(T, nkv, dv)
        want = np.zeros((T, nh, dv))
        for h in range(nh):
            sc = q[:, h] @ k[:, h // 2].T * 0.2
            sc[np.triu_indices(T, 1)] = -np.inf
            m = np.maximum(sc.max(-1, keepdims=True), f32(sink)[h])
            e = np.exp(sc - m)
            want[:, h] = (e / (e.sum(-1, keepdims=True) + np.exp(f32(sink)[h] - m))) @ v[:, h // 2]
            want[:, h] *= 1.0 / (1.0 + np.exp(-p32[:, nq + nk + nv + h]))[:, None]
        out = torch.empty(T, nh * dv, device="cuda", dtype=dtype)
        ops.gated_attention(q_out, pool, D(table), D(pos), D(slots), D(sink), D(proj), out, nh, nkv, dk, dv, 0.2,
                            gate_col=nq + nk + nv, gate_mode=2)
        fails += _say(f"attention with a sink and a gate, {str(dtype).split('.')[-1]}", float(np.abs(_f64(out).reshape(T, nh, dv) - want).max()), tol)
    # linear attention with a decay: 150 tokens whole and in chunks of 64
    heads, dk, dv, T = 2, 32, 48, 150
    nq, nv = heads * dk, heads * dv
    proj, decay = rng.normal(size=(T, 2 * nq + nv)) * 0.8, np.array([0.97, 0.6])
    silu = lambda z: z / (1.0 + np.exp(-z))
    p32 = f32(proj)
    q, k, v = silu(p32[:, :nq]).reshape(T, heads, dk), silu(p32[:, nq:2 * nq]).reshape(T, heads, dk), silu(p32[:, 2 * nq:]).reshape(T, heads, dv)
    want, St = np.zeros((T, heads, dv)), np.zeros((heads, dk, dv))
    for t in range(T):
        for h in range(heads):
            St[h] = f32(decay)[h] * St[h] + np.outer(k[t, h], v[t, h])
            want[t, h] = St[h].T @ q[t, h]
    entries = D(np.array([[0, T, 0, 0]], dtype=np.int32))
    for name, extra in (("whole", ()), ("in chunks", (D(np.array([[0, 0, 64, 1], [0, 64, 64, 0], [0, 128, 22, 2]], dtype=np.int32)),
                                                     D(np.array([[0, 3]], dtype=np.int32))))):
        state, o = torch.zeros(1, heads, dk * dv, device="cuda"), torch.empty(T, nv, device="cuda")
        ops.decay_scan(D(proj), D(decay), state, entries, o, heads, dk, dv, (0, nq, 2 * nq), *extra)
        fails += _say(f"linear attention with a decay, {name}", float(np.abs(_f64(o).reshape(T, heads, dv) - want).max()), 2e-5 * float(np.abs(want).max()))
        fails += _say(f"  its state, {name}", float(np.abs(_f64(state).reshape(heads, dk, dv) - St).max()), 2e-5 * float(np.abs(St).max()))
    return fails


def run_selftest() -> int:
    if not torch.cuda.is_available():
        print("[selftest] no GPU: the kernels of this framework run on an AMD GPU (gfx950) only", flush=True)
        return 1
    from .engine.engine import required_libraries
    from .ops.kernels import get_ops
    ops = get_ops()
    ops.preload(required_libraries("bfloat16"))
    rng = np.random.default_rng(1)
    fails = 0
    fails += case_linear(ops, rng)
    fails += case_rmsnorm(ops, rng)
    fails += case_rope(ops, rng)
    fails += case_attention(ops, rng, nh=4, nkv=2, hd=64, T=5, dtype=torch.float32)
    fails += case_attention(ops, rng, nh=4, nkv=2, hd=64, T=150, dtype=torch.bfloat16)
    fails += case_attention(ops, rng, nh=16, nkv=8, hd=128, T=2, dtype=torch.float32)
    fails += case_attention(ops, rng, nh=16, nkv=8, hd=128, T=300, dtype=torch.bfloat16)
    fails += case_attention(ops, rng, nh=3, nkv=1, hd=48, T=40, dtype=torch.bfloat16)
    fails += case_pointwise(ops, rng)
    fails += case_capped_attention(ops, rng, nh=4, nkv=2, dk=24, dv=40, T=70, dtype=torch.float32)
    fails += case_capped_attention(ops, rng, nh=6, nkv=1, dk=64, dv=16, T=130, dtype=torch.bfloat16)
    fails += case_mlstm(ops, rng, heads=2, dk=32, dv=48, lengths=[150, 1, 70], chunk=64)
    fails += case_mlstm(ops, rng, heads=1, dk=128, dv=128, lengths=[200], chunk=64)
    fails += case_norm_residual_and_experts(ops, rng)
    fails += case_diff_attention(ops, rng, nh=3, nkv=1, dk=20, dv=12, T=90, block=37, taps=3, rot=8, dtype=torch.float32, P=8)
    fails += case_diff_attention(ops, rng, nh=4, nkv=2, dk=32, dv=64, T=200, block=150, taps=4, rot=32, dtype=torch.bfloat16)
    fails += case_diff_attention(ops, rng, nh=8, nkv=1, dk=64, dv=128, T=130, block=64, taps=2, rot=16, dtype=torch.bfloat16)
    fails += case_streams_gates_and_decay(ops, rng)
    fails += case_embed_argmax_sample(ops, rng)
    fails += case_model_shapes(ops, rng)
    fails += case_head_bandwidth(ops, rng)
    print(f"[selftest] {'all cases passed' if fails == 0 else str(fails) + ' case(s) FAILED'}", flush=True)
    return fails


if __name__ == "__main__":
    sys.exit(run_selftest())
