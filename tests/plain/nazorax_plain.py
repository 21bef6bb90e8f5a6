"""A plain, slow implementation of the Nazorax decoder: whole sequences, no cache, no state
carried between calls, one function per mechanism, numpy float64.  It shares no code with the
engine: the tests compare the two.

The design in short.  x = E[token]; x0 is that embedding output.  Layers run in the listed
order; `loop` {start, stop, times} runs layers start .. stop - 1 `times` times in a row with the
same weights, and right before the first layer of every pass x <- W_in [x; x0].  A layer is
parallel: h = N(x), x <- x + mixer(h) + ff(h), N(x) = tanh(a x) * g + b with one learned number a
(no mean, no variance).  Mixers: sliding-window attention with grouped queries, biases on q, k, v
and a rotation of the first rot.dims entries of every head; latent attention, which keeps per token
a normed latent c and one rotated key part shared by all heads, forms every head's unrotated key and
value from c, rotates with YaRN-interpolated frequencies, is causal and has a learned sink in the
softmax's denominator.  Feed-forward: SwiGLU with biases, or routed experts with a clamped gated
activation (weights: softmax over the chosen logits) plus a shared expert.  Logits: head N(x).

`config` is the model's config.json as a dict, `w` maps tensor names to arrays.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import numpy as np


def rms_unit(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) along the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def dynamic_tanh(x: np.ndarray, w: Dict[str, np.ndarray], name: str) -> np.ndarray:
    return np.tanh(float(w[name + ".alpha"]) * x) * w[name] + w[name + ".b"]


def frequencies(rot: dict) -> tuple:
    """(frequency per pair, factor on cos and sin); YaRN's interpolation where rot has `scaling`."""
    dims, base = rot["dims"], rot["base"]
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)])
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def turns_to_dim(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turns_to_dim(sc["fast"])), 0)
    hi = min(math.ceil(turns_to_dim(sc["slow"])), dims - 1)
    ramp = np.clip((np.arange(half) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / sc["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(x: np.ndarray, positions: Sequence[int], rot: dict) -> np.ndarray:
    """x [T, ..., d]: the first rot.dims entries of the last axis are turned, entry i with entry i + dims/2."""
    dims = rot["dims"]
    half = dims // 2
    f, mag = frequencies(rot)
    out = x.copy()
    for t, p in enumerate(positions):
        a = p * f
        c, s = np.cos(a) * mag, np.sin(a) * mag
        u, v = x[t, ..., :half], x[t, ..., half:dims]
        out[t, ..., :half] = u * c - v * s
        out[t, ..., half:dims] = v * c + u * s
    return out


def window_mask(T: int, size: Optional[int]) -> np.ndarray:
    """visible[i, j]: 0 <= i - j < size (no size: every j <= i)."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    vis = j <= i
    if size:
        vis &= (i - j) < size
    return vis


def softmax_rows(s: np.ndarray, visible: np.ndarray, sink: Optional[float] = None) -> np.ndarray:
    """Softmax over the visible entries of each row; `sink` adds exp(sink) to the denominator only."""
    s = np.where(visible, s, -np.inf)
    top = s.max(axis=1, keepdims=True)
    if sink is not None:
        top = np.maximum(top, sink)
    p = np.exp(s - top)
    den = p.sum(axis=1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink - top)
    return p / den


def window_attention(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, m: dict) -> np.ndarray:
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = (h @ w[pre + ".q"].T + w[pre + ".q.b"]).reshape(T, H, d)
    k = (h @ w[pre + ".k"].T + w[pre + ".k.b"]).reshape(T, G, d)
    v = (h @ w[pre + ".v"].T + w[pre + ".v.b"]).reshape(T, G, dv)
    if m.get("rot") and m["rot"]["dims"]:
        q = rotate_half(q, range(T), m["rot"])
        k = rotate_half(k, range(T), m["rot"])
    visible = window_mask(T, m["mask"]["size"] if m.get("mask") else None)
    per = H // G
    out = np.zeros((T, H, dv))
    for hd in range(H):
        g = hd // per
        s = (q[:, hd, :] @ k[:, g, :].T) * m["scale"]
        out[:, hd, :] = softmax_rows(s, visible) @ v[:, g, :]
    return out.reshape(T, H * dv) @ w[pre + ".o"].T


def latent_attention(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, m: dict, eps: float) -> np.ndarray:
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[pre + ".q"].T).reshape(T, H, d + r)
    down = h @ w[pre + ".dkv"].T
    c = rms_unit(down[:, :rank], eps) * w[pre + ".dkv.norm"]
    k_rot = rotate_half(down[:, rank:], range(T), m["rot"])          # one rotated part, shared by all heads
    q_rot = rotate_half(q[:, :, d:], range(T), m["rot"])
    k_plain = (c @ w[pre + ".uk"].T).reshape(T, H, d)
    v = (c @ w[pre + ".uv"].T).reshape(T, H, dv)
    visible = window_mask(T, None)
    out = np.zeros((T, H, dv))
    for hd in range(H):
        s = (q[:, hd, :d] @ k_plain[:, hd, :].T + q_rot[:, hd, :] @ k_rot.T) * m["scale"]
        out[:, hd, :] = softmax_rows(s, visible, float(w[pre + ".sink"][hd])) @ v[:, hd, :]
    return out.reshape(T, H * dv) @ w[pre + ".o"].T


def silu(z: np.ndarray) -> np.ndarray:
    return z / (1.0 + np.exp(-z))


def dense_ff(h: np.ndarray, w: Dict[str, np.ndarray], pre: str) -> np.ndarray:
    g = h @ w[pre + ".gate"].T + w[pre + ".gate.b"]
    u = h @ w[pre + ".up"].T + w[pre + ".up.b"]
    return (silu(g) * u) @ w[pre + ".down"].T + w[pre + ".down.b"]


def clamped_expert(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, limit: float) -> np.ndarray:
    g = np.minimum(h @ w[pre + ".gate"].T, limit)
    u = np.clip(h @ w[pre + ".up"].T, -limit, limit)
    y = g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)
    return y @ w[pre + ".down"].T


def router_choice(h: np.ndarray, w_router: np.ndarray, top: int) -> tuple:
    """(indices [T, top], weights [T, top]): the largest logits (ties: the lower index), softmax over the chosen."""
    z = h @ w_router.T
    idx = np.argsort(-z, axis=1, kind="stable")[:, :top]
    chosen = np.take_along_axis(z, idx, axis=1)
    e = np.exp(chosen - chosen.max(axis=1, keepdims=True))
    return idx, e / e.sum(axis=1, keepdims=True)


def moe(h: np.ndarray, w: Dict[str, np.ndarray], pre: str, mlp: dict) -> np.ndarray:
    idx, wt = router_choice(h, w[pre + ".router"], mlp["router"]["top"])
    out = np.zeros((h.shape[0], w[pre + ".e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, s in zip(idx[t], wt[t]):
            out[t] += s * clamped_expert(h[t:t + 1], w, f"{pre}.e{e}", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out += clamped_expert(h, w, pre + ".shared", mlp["shared"]["limit"])
    return out


def run_order(config: dict) -> list:
    """[(layer index, True if a pass of the loop starts in front of it)]"""
    L = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(L)]
    order = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        order += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], L)]


def forward(config: dict, w: Dict[str, np.ndarray], tokens: Sequence[int], layers_out: Optional[list] = None) -> np.ndarray:
    """Logits [T, vocab] of a whole sequence from position 0."""
    eps = config["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    x0 = x.copy()
    for i, first_of_pass in run_order(config):
        layer, pre = config["layers"][i], f"l{i}"
        if first_of_pass:
            x = np.concatenate([x, x0], axis=1) @ w["loop.in"].T
        h = dynamic_tanh(x, w, pre + ".norm1")
        if layer["type"] == "attention":
            y = window_attention(h, w, pre + ".mix", layer["mixer"])
        elif layer["type"] == "latent_attention":
            y = latent_attention(h, w, pre + ".mix", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp:
            y = y + (dense_ff(h, w, pre + ".mlp") if mlp.get("kind", "dense") == "dense" else moe(h, w, pre + ".mlp", mlp))
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    return dynamic_tanh(x, w, "final.norm") @ w["head"].T
