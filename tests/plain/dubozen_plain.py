"""A plain, slow implementation of the Dubozen decoder: whole sequences, no cache, no state
carried between calls, one function per mechanism, numpy float64.  It shares no code with the
engine: the tests compare the two.

The design in short.  x = LN(E[token]) (LN: a layer norm with a gain and no bias).  The residual
is kept in `streams` copies (hyper-connections): a sublayer reads u = sum_s a_s x_s through LN and
its output y goes back as x_t <- sum_s B[s, t] x_s + c_t y; without `streams` there is one x and
x <- x + y.  A layer is mixer then feed-forward, each behind its own LN.  Mixers: `attention`
(grouped queries, a rotation of the first rot.dims entries of a head, a learned sink in the
softmax's denominator, values mixed with the values of the first such layer, an element-wise
sigmoid gate on the heads' outputs) and `parallel`: a softmax attention whose values are its keys
as projected (per-head RMS norms on q and k before the rotation, one gate number a head) beside a
linear attention with a fixed decay per head (S <- d S + k v^T, o = S^T q on silu'd projections,
one RMS norm over all heads, a sigmoid gate), the two added with fixed factors.  Feed-forward:
down(gelu_tanh(gate h) * up h), or routed experts (sigmoid scores, a correction added for the
choice only, groups of neighbouring experts of which the best are kept, weights renormalised and
scaled).  Logits: E LN(sum of the streams).

`config` is the model's config.json as a dict, `w` maps tensor names to arrays.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import numpy as np


def layer_norm(x: np.ndarray, g: np.ndarray, eps: float) -> np.ndarray:
    """(x - mean) / sqrt(var + eps) * g along the last axis, var the mean squared deviation."""
    mu = np.mean(x, axis=-1, keepdims=True)
    d = x - mu
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * g


def rms_norm(x: np.ndarray, g: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * g


def sigmoid(z: np.ndarray) -> np.ndarray:
    return 1.0 / (1.0 + np.exp(-z))


def silu(z: np.ndarray) -> np.ndarray:
    return z * sigmoid(z)


def gelu_tanh(z: np.ndarray) -> np.ndarray:
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half(x: np.ndarray, positions: Sequence[int], rot: Optional[dict]) -> np.ndarray:
    """x [T, heads, d]: entry i of the first rot.dims turns with entry i + dims/2 by p * base^(-2i/dims)."""
    if not rot or not rot.get("dims"):
        return x
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    out = x.copy()
    for t, p in enumerate(positions):
        c, s = np.cos(p * f), np.sin(p * f)
        u, v = x[t, :, :half], x[t, :, half:dims]
        out[t, :, :half] = u * c - v * s
        out[t, :, half:dims] = v * c + u * s
    return out


def causal_softmax(scores: np.ndarray, sink: Optional[float] = None) -> np.ndarray:
    """scores [T, T] -> weights; row i sees columns j <= i; exp(sink) joins the denominator only."""
    T = scores.shape[0]
    vis = np.tril(np.ones((T, T), dtype=bool))
    s = np.where(vis, scores, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink)
    e = np.exp(s - m)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink - m)
    return e / den


def softmax_heads(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, sink: Optional[np.ndarray]) -> np.ndarray:
    """q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]; query head h reads kv head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // (H // G)
        p = causal_softmax(q[:, h] @ k[:, g].T * scale, None if sink is None else float(sink[h]))
        out[:, h] = p @ v[:, g]
    return out


def sink_attention(h: np.ndarray, positions, m: dict, w: Dict[str, np.ndarray], name: str, v_first: Optional[np.ndarray]):
    """The mixer `attention`.  Returns (output [T, width], the values it cached [T, G, dv])."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = (h @ w[name + ".q"].T).reshape(T, H, d)
    k = (h @ w[name + ".k"].T).reshape(T, G, d)
    v = (h @ w[name + ".v"].T).reshape(T, G, dv)
    q = rotate_half(q, positions, m.get("rot"))
    k = rotate_half(k, positions, m.get("rot"))
    if v_first is not None:
        lam = float(w[name + ".vmix"])
        v = (1.0 - lam) * v + lam * v_first
    o = softmax_heads(q, k, v, m["scale"], w[name + ".sink"])
    o = o.reshape(T, H * dv) * sigmoid(h @ w[name + ".g"].T)
    return o @ w[name + ".o"].T, v


def keyed_attention(h: np.ndarray, positions, m: dict, w: Dict[str, np.ndarray], name: str, eps: float) -> np.ndarray:
    """The left half of `parallel`: values are the keys as projected; norms on q and k; one gate a head."""
    T = h.shape[0]
    H, G, d = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    q = (h @ w[name + ".q"].T).reshape(T, H, d)
    k = (h @ w[name + ".k"].T).reshape(T, G, d)
    v = k.copy()
    q = rotate_half(rms_norm(q, w[name + ".q.norm"], eps), positions, m.get("rot"))
    k = rotate_half(rms_norm(k, w[name + ".k.norm"], eps), positions, m.get("rot"))
    o = softmax_heads(q, k, v, m["scale"], None)
    o = o * sigmoid(h @ w[name + ".g"].T)[:, :, None]
    return o.reshape(T, H * d) @ w[name + ".o"].T


def decayed_linear_attention(h: np.ndarray, m: dict, w: Dict[str, np.ndarray], name: str, eps: float) -> np.ndarray:
    """The right half of `parallel`, token by token: S <- decay S + k v^T, o = S^T q."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = silu(h @ w[name + ".q"].T).reshape(T, H, d)
    k = silu(h @ w[name + ".k"].T).reshape(T, H, d)
    v = silu(h @ w[name + ".v"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for j in range(H):
        S = np.zeros((d, dv))
        for t in range(T):
            S = m["decay"][j] * S + np.outer(k[t, j], v[t, j])
            o[t, j] = S.T @ q[t, j]
    o = rms_norm(o.reshape(T, H * dv), w[name + ".norm"], eps) * sigmoid(h @ w[name + ".g"].T)
    return o @ w[name + ".o"].T


def parallel_mixer(h, positions, m, w, name, eps):
    left = keyed_attention(h, positions, m["left"], w, name + ".left", eps)
    right = decayed_linear_attention(h, m["right"], w, name + ".right", eps)
    return m["left_scale"] * left + m["right_scale"] * right


def dense_ff(h: np.ndarray, w: Dict[str, np.ndarray], name: str) -> np.ndarray:
    return (gelu_tanh(h @ w[name + ".gate"].T) * (h @ w[name + ".up"].T)) @ w[name + ".down"].T


def route(h: np.ndarray, r: dict, w: Dict[str, np.ndarray], name: str):
    """(chosen experts [T, top], weights [T, top]) of the grouped sigmoid router."""
    T = h.shape[0]
    E, top = r["experts"], r["top"]
    s = sigmoid(h @ w[name + ".router"].T)
    choice = s + w[name + ".correction"]
    groups = r.get("groups")
    if groups:
        n, keep = groups["count"], groups["keep"]
        per = E // n
        allowed = np.zeros((T, E), dtype=bool)
        for t in range(T):
            gs = []
            for g in range(n):
                c = np.sort(choice[t, g * per:(g + 1) * per])[::-1]
                gs.append(c[:2].sum())
            for g in np.argsort(-np.array(gs), kind="stable")[:keep]:
                allowed[t, g * per:(g + 1) * per] = True
        choice = np.where(allowed, choice, -np.inf)
    ids = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    chosen = np.take_along_axis(s, ids, axis=-1)
    wts = chosen / (chosen.sum(axis=-1, keepdims=True) + 1e-20) * r.get("scale", 1.0)
    return ids, wts


def expert_ff(h: np.ndarray, mlp: dict, w: Dict[str, np.ndarray], name: str) -> np.ndarray:
    ids, wts = route(h, mlp["router"], w, name)
    out = np.zeros((h.shape[0], w[name + ".e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, a in zip(ids[t], wts[t]):
            p = f"{name}.e{e}"
            out[t] += a * ((silu(h[t] @ w[p + ".gate"].T) * (h[t] @ w[p + ".up"].T)) @ w[p + ".down"].T)
    return out


def forward(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int], trace: Optional[List[np.ndarray]] = None) -> np.ndarray:
    """Logits [T, vocab] of one sequence from position 0.  `trace` collects the residual (summed over the streams) after every layer."""
    w = {k: np.asarray(v, dtype=np.float64) for k, v in w.items()}
    eps = config["norm"]["eps"]
    T = len(tokens)
    positions = list(range(T))
    x0 = layer_norm(w["embed"][np.asarray(tokens)], w["embed.norm"], eps)
    S = config.get("streams")
    xs = [x0.copy() for _ in range(S or 1)]
    v_first = None
    seen_first = False

    def sublayer(q: int, name: str, fn):
        nonlocal xs
        if S:
            a, c, B = w[f"{name}.hc{q}.in"], w[f"{name}.hc{q}.out"], w[f"{name}.hc{q}.mix"]
            u = sum(a[s] * xs[s] for s in range(S))
        else:
            u = xs[0]
        y = fn(layer_norm(u, w[f"{name}.norm{q}"], eps))
        if S:
            xs = [sum(B[s, t] * xs[s] for s in range(S)) + c[t] * y for t in range(S)]
        else:
            xs = [xs[0] + y]

    for i, layer in enumerate(config["layers"]):
        name = f"l{i}"
        m = layer["mixer"]
        if layer["type"] == "attention":
            def mix(h, m=m, name=name):
                nonlocal v_first, seen_first
                mixing = bool(m.get("v_mix"))
                y, v = sink_attention(h, positions, m, w, name + ".mix", v_first if (mixing and seen_first) else None)
                if mixing and not seen_first:
                    v_first, seen_first = v, True
                return y
        elif layer["type"] == "parallel":
            def mix(h, m=m, name=name):
                return parallel_mixer(h, positions, m, w, name + ".mix", eps)
        else:
            raise ValueError(layer["type"])
        sublayer(1, name, mix)
        mlp = layer.get("mlp")
        if mlp:
            if mlp["kind"] == "dense":
                sublayer(2, name, lambda h, name=name: dense_ff(h, w, name + ".mlp"))
            else:
                sublayer(2, name, lambda h, name=name, mlp=mlp: expert_ff(h, mlp, w, name + ".mlp"))
        if trace is not None:
            trace.append(sum(xs))
    x = sum(xs)
    return layer_norm(x, w["final.norm"], eps) @ w["embed"].T
