"""Small Nazorax configurations and random weights for the tests.  The weights are drawn here with numpy (not by the
framework's own generator), rounded to bfloat16 and written with the safetensors package, so that the engine and the
plain implementation read the same numbers.  Scales are chosen so that activations stay of order one, attention is far
from uniform, the sinks matter, the clamps of the experts' activation bite, and the Dynamic Tanh is neither linear nor
saturated."""
import json
import os

import numpy as np


def yarn(factor, original, fast, slow):
    return dict(factor=factor, original=original, fast=fast, slow=slow)


def attention(heads, kv_heads, dim, vdim, scale, window, rot_dims, base=10000.0, mlp=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=dict(base=base, dims=rot_dims))
    if window:
        m["mask"] = dict(size=window)
    return dict(type="attention", mixer=m, mlp=mlp)


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, scaling=None, mlp=None):
    rot = dict(base=base, dims=rot_dim)
    if scaling:
        rot["scaling"] = scaling
    return dict(type="latent_attention", mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale, rot=rot), mlp=mlp)


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, limit, shared_ff=None, shared_limit=None):
    d = dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))
    if shared_ff:
        d["shared"] = dict(ff=shared_ff, limit=shared_limit)
    return d


CONFIGS = {
    # a loop of two layers taken three times in the middle; three query heads over one kv head with a window of 21 that is no
    # multiple of a page; the rotation on part of a head; a latent layer with YaRN; experts with and without a shared one
    "looped": dict(architecture="Nazorax", width=48, vocab=97, norm=dict(eps=1e-5), loop=dict(start=1, stop=3, times=3),
                   layers=[attention(3, 1, 16, 24, 0.25, 21, 8, 1000.0, mlp=dense(72)),
                           latent(2, 12, 8, 10, 24, 0.2, 500.0, yarn(4.0, 32, 8.0, 1.0), mlp=moe(5, 2, 20, 1.2, 28, 0.9)),
                           attention(4, 2, 8, 8, 0.35, 40, 8, 100.0, mlp=moe(3, 3, 16, 2.5)),
                           latent(3, 8, 4, 16, 20, 0.3, 10000.0, None, mlp=dense(40))]),
    # sizes that are no multiples of 4 or 16; a loop from the first layer on, taken once; a layer without a feed-forward; one
    # head; every head its own kv head; no rotation at all in one layer; a window longer than any request; one expert of one;
    # a latent head without unrotated entries' majority (dim 2 beside rot 6)
    "odd": dict(architecture="Nazorax", width=50, vocab=61, norm=dict(eps=3e-6), loop=dict(start=0, stop=2, times=1),
                layers=[latent(1, 2, 6, 7, 9, 0.4, 50.0, yarn(8.0, 16, 4.0, 0.5), mlp=moe(1, 1, 9, 3.0, 5, 0.5)),
                        attention(5, 5, 6, 10, 0.5, 1000, 0, 10000.0, mlp=None),
                        attention(2, 2, 10, 7, 0.3, 7, 10, 20.0, mlp=moe(7, 4, 21, 0.8))]),
    # no loop; widths the matrix-core kernels serve: keys and values of 64 under a window of 50, pages of 16, experts of 96
    "wide": dict(architecture="Nazorax", width=128, vocab=320, norm=dict(eps=1e-6),
                 layers=[attention(4, 2, 64, 64, 0.125, 50, 32, 30000.0, mlp=moe(8, 2, 96, 1.5, 160, 1.0)),
                         latent(4, 32, 16, 32, 64, 0.15, 10000.0, yarn(3.0, 64, 16.0, 1.0), mlp=dense(160)),
                         attention(2, 1, 32, 32, 0.18, 0, 32, 10000.0, mlp=moe(6, 1, 32, 2.0))]),
}


def to_bf16(a):
    import torch
    a = np.asarray(a, dtype=np.float32)
    return torch.from_numpy(np.ascontiguousarray(a)).reshape(a.shape).to(torch.bfloat16)      # a single number keeps its shape ()


def draw_weights(config, seed):
    """{name: torch bfloat16 tensor} for every tensor the configuration's model holds."""
    rng = np.random.default_rng(seed)
    W, V = config["width"], config["vocab"]
    t = {}

    def mat(rows, cols, gain=1.0):
        return rng.normal(0.0, gain / np.sqrt(cols), size=(rows, cols))

    def norm(name):
        t[name] = 1.0 + rng.normal(0.0, 0.2, size=W)
        t[name + ".b"] = rng.normal(0.0, 0.2, size=W)
        t[name + ".alpha"] = np.asarray(rng.uniform(0.3, 0.8))

    def gated(pre, F, bias):
        t[pre + ".gate"] = mat(F, W, 2.0)
        t[pre + ".up"] = mat(F, W, 2.0)
        t[pre + ".down"] = mat(W, F)
        if bias:
            t[pre + ".gate.b"] = rng.normal(0.0, 0.3, size=F)
            t[pre + ".up.b"] = rng.normal(0.0, 0.3, size=F)
            t[pre + ".down.b"] = rng.normal(0.0, 0.3, size=W)

    t["embed"] = rng.normal(0.0, 1.0, size=(V, W))
    t["head"] = mat(V, W)
    norm("final.norm")
    if config.get("loop"):
        t["loop.in"] = mat(W, 2 * W, 1.4)
    for i, lay in enumerate(config["layers"]):
        p, m = f"l{i}", lay["mixer"]
        norm(p + ".norm1")
        H = m["heads"]
        if lay["type"] == "attention":
            G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
            for name, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
                t[f"{p}.mix.{name}"] = mat(rows, W, 2.0 if name != "v" else 1.0)
                t[f"{p}.mix.{name}.b"] = rng.normal(0.0, 0.4, size=rows)
            t[p + ".mix.o"] = mat(W, H * dv)
        else:
            d, r, dv, R = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            t[p + ".mix.q"] = mat(H * (d + r), W, 2.0)
            t[p + ".mix.dkv"] = mat(R + r, W, 2.0)
            t[p + ".mix.dkv.norm"] = 1.0 + rng.normal(0.0, 0.3, size=R)
            t[p + ".mix.uk"] = mat(H * d, R, 1.5)
            t[p + ".mix.uv"] = mat(H * dv, R)
            t[p + ".mix.sink"] = rng.normal(0.5, 1.0, size=H)
            t[p + ".mix.o"] = mat(W, H * dv)
        mlp = lay.get("mlp")
        if mlp and mlp["kind"] == "dense":
            gated(p + ".mlp", mlp["ff"], True)
        elif mlp:
            E = mlp["router"]["experts"]
            t[p + ".mlp.router"] = mat(E, W, 2.0)
            for e in range(E):
                gated(f"{p}.mlp.e{e}", mlp["expert"]["ff"], False)
            if mlp.get("shared"):
                gated(p + ".mlp.shared", mlp["shared"]["ff"], False)
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
