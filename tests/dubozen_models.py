"""Small Dubozen configurations and random weights for the tests.  The weights are drawn here with numpy (not by the
framework's own generator), rounded to bfloat16 and written with the safetensors package, so that the engine and the
plain implementation read the same numbers.  Scales are chosen so that activations stay of order one, attention is far
from uniform, the sinks and the corrections of the routers matter, and the streams neither die out nor blow up."""
import json
import os

import numpy as np


def softmax_attention(heads, kv_heads, dim, vdim, scale, rot_dims, base=10000.0):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if rot_dims is not None:
        m["rot"] = dict(base=base, dims=rot_dims)
    return m


def attention(heads, kv_heads, dim, vdim, scale, rot_dims, base=10000.0, v_mix=False, mlp=None):
    m = softmax_attention(heads, kv_heads, dim, vdim, scale, rot_dims, base)
    m["v_mix"] = v_mix
    return dict(type="attention", mixer=m, mlp=mlp)


def parallel(left, right_heads, right_dim, right_vdim, decay, left_scale, right_scale, mlp=None):
    return dict(type="parallel", mlp=mlp,
                mixer=dict(left=left, right=dict(heads=right_heads, dim=right_dim, vdim=right_vdim, decay=list(decay)),
                           left_scale=left_scale, right_scale=right_scale))


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, scale, groups=None, keep=None):
    r = dict(experts=experts, top=top, scale=scale)
    if groups:
        r["groups"] = dict(count=groups, keep=keep)
    return dict(kind="moe", expert=dict(ff=ff), router=r)


CONFIGS = {
    # three streams; two attention layers that mix their values and one that does not; rotation on part of a head, on all of it;
    # two kv heads under four heads, one under two; experts in three groups of which two are kept; a layer without a feed-forward
    "streams": dict(architecture="Dubozen", width=48, vocab=97, norm=dict(eps=1e-5), streams=3,
                    layers=[attention(4, 2, 16, 24, 0.25, 8, 1000.0, v_mix=True, mlp=dense(72)),
                            parallel(softmax_attention(4, 2, 8, 8, 0.4, 8, 100.0), 3, 8, 12, [0.5, 0.9, 0.995], 0.7, 0.4,
                                     mlp=moe(6, 2, 20, 1.7, 3, 2)),
                            attention(2, 2, 12, 24, 0.3, 4, 500.0, v_mix=True, mlp=None),
                            parallel(softmax_attention(2, 1, 16, 16, 0.25, 6, 10000.0), 2, 12, 8, [0.97, 0.8], 1.2, 0.9, mlp=dense(40)),
                            attention(3, 1, 8, 10, 0.35, 8, 50.0, v_mix=False, mlp=moe(4, 1, 16, 0.8))]),
    # one residual (no streams at all); sizes that are no multiples of 4; the first layer parallel; every head its own kv head; one
    # head; no rotation in one layer; one expert of one; a single layer that keeps its values for nobody; a layer without a
    # feed-forward; groups of one expert each
    "plain": dict(architecture="Dubozen", width=50, vocab=61, norm=dict(eps=3e-6),
                  layers=[parallel(softmax_attention(3, 3, 6, 6, 0.5, 2, 20.0), 1, 5, 7, [0.93], 1.0, 1.0, mlp=moe(1, 1, 9, 2.0)),
                          attention(5, 5, 10, 7, 0.3, None, v_mix=True, mlp=None),
                          parallel(softmax_attention(1, 1, 10, 10, 0.3, 10, 30.0), 3, 6, 6, [0.999, 0.3, 0.75], 0.5, 1.5,
                                   mlp=moe(5, 2, 21, 1.0, 5, 3)),
                          attention(2, 1, 6, 9, 0.45, 0, v_mix=False, mlp=dense(33))]),
    # sizes the matrix cores serve: keys and values of 64 and 32, pages of 16, four streams, states of 64 x 64
    "wide": dict(architecture="Dubozen", width=128, vocab=320, norm=dict(eps=1e-6), streams=4,
                 layers=[parallel(softmax_attention(4, 1, 64, 64, 0.125, 32, 30000.0), 2, 64, 64, [0.9, 0.99], 0.8, 0.6, mlp=dense(160)),
                         attention(4, 2, 64, 64, 0.125, 64, 10000.0, v_mix=True, mlp=moe(8, 3, 64, 2.0, 4, 2)),
                         attention(8, 2, 32, 64, 0.18, 16, 10000.0, v_mix=True, mlp=dense(96)),
                         parallel(softmax_attention(2, 2, 32, 32, 0.18, 16, 10000.0), 4, 32, 32, [0.6, 0.8, 0.95, 0.999], 0.6, 0.5,
                                  mlp=moe(6, 1, 32, 1.0))]),
    # keys of 32 over values of 16 (padded to 32 in the pages) and keys and values of 128 under a sink (the other two sizes the
    # matrix cores serve), two streams
    "squares": dict(architecture="Dubozen", width=64, vocab=100, norm=dict(eps=1e-6), streams=2,
                    layers=[attention(4, 1, 32, 16, 0.2, 32, 10000.0, v_mix=False, mlp=dense(48)),
                            attention(2, 2, 128, 128, 0.09, 64, 10000.0, v_mix=False, mlp=None),
                            parallel(softmax_attention(4, 2, 128, 128, 0.09, 32, 10000.0), 1, 128, 128, [0.98], 0.7, 0.7, mlp=moe(4, 2, 32, 1.5, 2, 1)),
                            parallel(softmax_attention(2, 1, 32, 32, 0.2, 8, 100.0), 2, 16, 48, [0.9, 0.7], 1.0, 0.5, mlp=dense(64))]),
    # one stream kept as streams (hyper-connections of one copy)
    "single": dict(architecture="Dubozen", width=32, vocab=40, norm=dict(eps=1e-5), streams=1,
                   layers=[attention(2, 1, 8, 8, 0.35, 4, 100.0, v_mix=False, mlp=dense(24)),
                           parallel(softmax_attention(2, 2, 8, 8, 0.35, 8, 100.0), 2, 4, 4, [0.9, 0.5], 1.0, 1.0, mlp=None)]),
}


def to_bf16(a):
    import torch
    a = np.asarray(a, dtype=np.float32)
    return torch.from_numpy(np.ascontiguousarray(a)).reshape(a.shape).to(torch.bfloat16)      # a single number keeps its shape ()


def draw_weights(config, seed):
    """{name: torch bfloat16 tensor} for every tensor the configuration's model holds."""
    rng = np.random.default_rng(seed)
    W, V, S = config["width"], config["vocab"], config.get("streams")
    t = {}

    def mat(rows, cols, gain=1.0):
        return rng.normal(0.0, gain / np.sqrt(cols), size=(rows, cols))

    def norm(name, n=W):
        t[name] = 1.0 + rng.normal(0.0, 0.2, size=n)

    def gated(pre, F):
        t[pre + ".gate"] = mat(F, W, 2.0)
        t[pre + ".up"] = mat(F, W, 2.0)
        t[pre + ".down"] = mat(W, F)

    def softmax_part(pre, m, with_v):
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t[pre + ".q"] = mat(H * d, W, 2.0)
        t[pre + ".k"] = mat(G * d, W, 2.0)
        if with_v:
            t[pre + ".v"] = mat(G * dv, W)
        t[pre + ".o"] = mat(W, H * dv)

    t["embed"] = rng.normal(0.0, 1.0, size=(V, W))
    norm("embed.norm")
    norm("final.norm")
    for i, lay in enumerate(config["layers"]):
        p, m = f"l{i}", lay["mixer"]
        norm(p + ".norm1")
        if lay["type"] == "attention":
            softmax_part(p + ".mix", m, True)
            t[p + ".mix.g"] = mat(m["heads"] * m["vdim"], W, 1.5)
            t[p + ".mix.sink"] = rng.normal(0.5, 1.0, size=m["heads"])
            if m.get("v_mix"):
                t[p + ".mix.vmix"] = np.asarray(rng.uniform(0.25, 0.6))
        else:
            left, right = m["left"], m["right"]
            softmax_part(p + ".mix.left", left, False)
            t[p + ".mix.left.q.norm"] = 1.0 + rng.normal(0.0, 0.3, size=left["dim"])
            t[p + ".mix.left.k.norm"] = 1.0 + rng.normal(0.0, 0.3, size=left["dim"])
            t[p + ".mix.left.g"] = mat(left["heads"], W, 1.5)
            H, d, dv = right["heads"], right["dim"], right["vdim"]
            t[p + ".mix.right.q"] = mat(H * d, W, 1.5)
            t[p + ".mix.right.k"] = mat(H * d, W, 1.5)
            t[p + ".mix.right.v"] = mat(H * dv, W, 1.5)
            t[p + ".mix.right.g"] = mat(H * dv, W, 1.5)
            t[p + ".mix.right.o"] = mat(W, H * dv)
            norm(p + ".mix.right.norm", H * dv)
        mlp = lay.get("mlp")
        if mlp:
            norm(p + ".norm2")
        if mlp and mlp["kind"] == "dense":
            gated(p + ".mlp", mlp["ff"])
        elif mlp:
            E = mlp["router"]["experts"]
            t[p + ".mlp.router"] = mat(E, W, 2.0)
            t[p + ".mlp.correction"] = rng.normal(0.0, 0.3, size=E)
            for e in range(E):
                gated(f"{p}.mlp.e{e}", mlp["expert"]["ff"])
        if S:
            for q in (1, 2) if mlp else (1,):
                t[f"{p}.hc{q}.in"] = 1.0 / S + rng.normal(0.0, 0.15, size=S)
                t[f"{p}.hc{q}.out"] = 1.0 + rng.normal(0.0, 0.3, size=S)
                t[f"{p}.hc{q}.mix"] = np.eye(S) + rng.normal(0.0, 0.15, size=(S, S))
    return {k: to_bf16(v) for k, v in t.items()}


def write_folder(path, config, seed, weights=None):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    w = weights if weights is not None else draw_weights(config, seed)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return path


def as_float64(weights):
    import torch
    return {k: v.to(torch.float64).numpy() for k, v in weights.items()}
