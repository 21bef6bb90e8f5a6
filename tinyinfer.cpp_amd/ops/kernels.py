"""The kernels, as Python calls on torch tensors.

Each call hands its tensors to the host library's `Ops` (ops/ops.cpp), which
checks devices, dtypes and shapes, picks the kernel for the sizes, and launches
the hand-written HIP kernel through the C interface of the kernel libraries
(`csrc/`).  Nothing here computes with torch, and nothing falls back to the CPU or
to a library: without a GPU or without the compiled libraries a call raises.
`Ops.lib(name)` gives a kernel library itself, for tests that call one kernel.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Optional

from .. import native
from ..csrc import build as _build
from ..native import KernelError  # noqa: F401

F32, BF16 = 0, 1
EPI = {"store": 0, "add": 1, "store_act": 2, "swiglu": 3}

_C_TYPES = {"int": ctypes.c_int, "long": ctypes.c_long, "float": ctypes.c_float, "unsigned long": ctypes.c_ulong}


def required_libraries(dtype: str):
    """The kernel libraries a model of this dtype needs (what a first call compiles)."""
    return _build.libraries_for(dtype)


def header_signatures(text: str) -> Dict[str, tuple]:
    """{function: (restype, [argtypes])} of the `int ti_...(...)`, `long ti_...(...)` and `void ti_...(...)`
    declarations of a kernels' header: pointers and streams as void pointers, int, long and
    float as themselves.  A declaration with any other type raises."""
    import re
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for ret, name, args in re.findall(r"\b(int|long|void)\s+(ti_\w+)\s*\(([^)]*)\)\s*;", text):
        types = []
        for arg in (a.strip() for a in args.split(",")):
            if not arg or arg == "void":
                continue
            if "*" in arg or arg.startswith("hipStream_t"):
                types.append(ctypes.c_void_p)
                continue
            words = [w for w in arg.replace("const", " ").split()]
            kind = " ".join(words[:-1])
            if len(words) < 2 or kind not in _C_TYPES:
                raise KernelError(f"tinyinfer_kernels.h: cannot read the argument {arg!r} of {name}")
            types.append(_C_TYPES[kind])
        out[name] = ({"int": ctypes.c_int, "long": ctypes.c_long, "void": None}[ret], types)
    return out


_signatures: Optional[Dict[str, tuple]] = None


def declare_signatures(lib: ctypes.CDLL) -> None:
    """Give every function of the headers that this library exports its argument types."""
    global _signatures
    if _signatures is None:
        _signatures = {}
        for header in ("tinyinfer_kernels.h", "tinyinfer_kernels_tuning.h"):
            with open(os.path.join(_build.HERE, header)) as f:
                _signatures.update(header_signatures(f.read()))
    for name, (restype, argtypes) in _signatures.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            continue
        fn.restype = restype
        fn.argtypes = argtypes


class NormedRows:
    """rmsnorm(x; weight, eps) that has not been computed yet: `Ops.linear` accepts it in place of
    the activation and runs the norm inside the product's kernel where a kernel for that exists,
    else it computes the rows into `out` first."""

    def __init__(self, x, weight, eps: float, out):
        self.x, self.weight, self.eps, self.out = x, weight, eps, out
        self.shape = out.shape
        self.dtype = out.dtype

    def materialize(self, ops: "Ops"):
        ops.rmsnorm(self.x, self.weight, self.eps, self.out)
        return self.out


_SWITCHES = {"use_fast_gemm": "fast_gemm", "use_fast_attention": "fast_attention", "use_fused_norm": "fused_norm",
             "use_fused_qk_decode": "fused_qk_decode", "use_fused_qkv_prefill": "fused_qkv_prefill",
             "use_split_k_add": "split_k_add", "use_deferred_add": "deferred_add", "use_paired_prefill": "paired_prefill",
             "use_portion_splits": "portion_splits", "use_early_page_ids": "early_page_ids",
             "use_radix_sample": "radix_sample", "use_shared_tiles": "shared_tiles"}
_LIB_OF = {"embed": "core", "rmsnorm": "core", "rope_neox": "core", "rope_table": "core", "qk_norm_rope_kv_write": "core",
           "qk_norm_inplace": "core", "argmax": "sampling", "sample": "sampling", "attention_rows": "attention_generic",
           "fill_random": "core", "fill_zero": "core", "add_sinusoid": "pointwise", "add_row": "pointwise", "xielu": "pointwise",
           "scaled_add": "pointwise", "qkv_split_write": "pointwise", "attention_capped": "attention_generic",
           "mlstm_scan": "recurrent", "gated_head_norm": "recurrent", "norm_residual": "residual", "round_rows": "residual",
           "scale": "residual", "short_conv": "diff_attention", "diff_qk_prep": "diff_attention", "diff_attention": "diff_attention",
           "moe_route": "moe", "moe_experts": "moe", "moe_experts_gated": "moe", "qkv_prep_write": "pointwise", "dyt": "pointwise",
           "gated_act": "pointwise", "concat_round": "pointwise", "latent_prep": "latent_attention",
           "latent_attention": "latent_attention", "latent_transpose": "latent_attention", "layernorm": "hyper",
           "layernorm_mixed": "hyper", "hyper_combine": "hyper", "hyper_spread": "hyper", "hyper_write": "hyper",
           "gated_qkv_prep": "gated_attention", "gated_attention": "gated_attention", "decay_scan": "linear_attention",
           "gated_row_norm": "linear_attention", "moe_route_grouped": "moe"}


class Ops:
    """One method per op, on an `Ops` object of the host library: an engine's own, or one made here."""

    def __init__(self, _borrowed: Optional[int] = None):
        object.__setattr__(self, "_libs", {})
        object.__setattr__(self, "_own", _borrowed is None)
        if _borrowed is None:
            t = native.torch()
            if not t.cuda.is_available():
                raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
            native.use_torch_allocator()
            _borrowed = native.pointer("ti_ops_create", None)
        object.__setattr__(self, "_ptr", _borrowed)

    def __del__(self):
        try:
            if self._own and native._lib is not None:
                native._lib.ti_ops_release(self._ptr)
        except Exception:  # noqa: BLE001
            pass

    # switches for tests and measurements (each leaves the results the same up to the order of sums)
    def __getattr__(self, name):
        if name in _SWITCHES:
            old = ctypes.c_int()
            native.call("ti_ops_switch", self._ptr, _SWITCHES[name].encode(), -1, ctypes.byref(old))
            if name in ("use_fast_gemm", "use_fast_attention"):
                lib = "gemm_bf16" if name == "use_fast_gemm" else "attention_bf16"
                return bool(old.value) and os.path.isfile(os.path.join(_build.HERE, _build.SOURCES[lib]))
            return bool(old.value)
        if name == "_pending":
            return type(self)._pending.fget(self)
        if name == "force_decode_splits":
            old = ctypes.c_int()
            native.call("ti_ops_switch", self._ptr, b"force_decode_splits", -1, ctypes.byref(old))
            return old.value
        if name == "force_paired_tiles":
            old = ctypes.c_int()
            native.call("ti_ops_switch", self._ptr, b"force_paired_tiles", -2, ctypes.byref(old))
            return None if old.value < 0 else bool(old.value)
        raise AttributeError(name)

    def __setattr__(self, name, value):
        if name in _SWITCHES:
            native.call("ti_ops_switch", self._ptr, _SWITCHES[name].encode(), int(bool(value)), None)
        elif name == "force_decode_splits":
            native.call("ti_ops_switch", self._ptr, b"force_decode_splits", int(value or 0), None)
        elif name == "force_paired_tiles":
            native.call("ti_ops_switch", self._ptr, b"force_paired_tiles", -1 if value is None else int(bool(value)), None)
        else:
            object.__setattr__(self, name, value)

    # ------------------------------------------------------------------ loading
    def lib(self, name: str) -> ctypes.CDLL:
        """A kernel library itself (the same one the host library has loaded)."""
        lib = self._libs.get(name)
        if lib is None:
            if not native.torch().cuda.is_available():
                raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
            native.ensure_kernels([name])
            lib = ctypes.CDLL(_build.find(name))
            lib.ti_last_error.restype = ctypes.c_char_p
            declare_signatures(lib)
            self._libs[name] = lib
        return lib

    def preload(self, names):
        """Compile (if needed, several at a time) and register the libraries `names`."""
        if not native.torch().cuda.is_available():
            raise KernelError("no GPU: the kernels of this framework run on an AMD GPU (gfx950) only")
        native.ensure_kernels(list(names))

    @staticmethod
    def _check(lib, rc, what):
        if rc != 0:
            raise KernelError(f"{what}: {lib.ti_last_error().decode()}")

    def _raw_stream(self):
        return None

    _stream = _raw_stream

    def _call(self, op: str, tensors=(), numbers=(), text: Optional[str] = None, fold=(), libs=()) -> int:
        native.ensure_kernels(libs or [_LIB_OF.get(op, "core")])
        for t in tensors:
            if t is not None and not t.is_cuda:
                raise KernelError("kernel arguments must live on the GPU")
        res = native.ti_tensor()
        nums = (ctypes.c_double * max(1, len(numbers)))(*[float(v) for v in numbers])
        native.call("ti_ops_call", self._ptr, op.encode(), native.describe_many(tensors, fold), len(tensors), nums,
                    len(numbers), native.enc(text), ctypes.byref(res))
        return res.shape[0]

    @property
    def _pending(self):
        """The number of partial sums a product left for the next norm (None: none are waiting)."""
        return self._call("pending", libs=["core"]) or None

    def timing(self, on: bool) -> None:
        """Switch per-call timing with events on or off (see `Ops::timing`)."""
        self._call("timing", [], [int(bool(on))], libs=["core"])

    def tune(self, library: Optional[str] = None, name: str = "", value: int = 0) -> None:
        """Force a shape rule of a kernel library for this object's calls (`Ops::tune`; the names are listed in
        csrc/tinyinfer_kernels_tuning.h).  Without arguments: every override of this object goes."""
        if library is None:
            self._call("tune", [], [0], libs=["core"])
        else:
            self._call("tune", [], [int(value)], text=f"{library} {name}", libs=[library])

    def count_calls(self, on: bool) -> None:
        """List the calls without timing them (see `Ops::count_calls`): a step runs exactly as it does unobserved;
        `timing_report()` then gives the names, each ending in what the call took ("[mfma]", "[generic]", "[fused]")."""
        self._call("count_calls", [], [int(bool(on))], libs=["core"])

    def timing_report(self):
        """[{"name", "calls", "us"}] of the calls since timing was switched on (or last reported)."""
        import json
        return json.loads(native.text("ti_ops_timing_report", self._ptr))

    def flush(self):
        """Partial sums that a product left for the next norm are added now (same bits).  Every launch
        through this object does it first; code that reads such a residual with torch calls it itself."""
        self._call("flush", libs=["core"])

    # --------------------------------------------------------------------- ops
    def embed(self, table, tokens, x):
        self._call("embed", [table, tokens, x])

    def rmsnorm(self, x, w, eps, out, rows=None):
        self._call("rmsnorm", [x, w, out, rows], [eps])

    def rope_neox(self, x, positions, inv_freq):
        """In place on f32 x [M, heads, hd]; the last two dims contiguous, rows may be strided."""
        self._call("rope_neox", [x, positions, inv_freq])

    def rope_table(self, inv_freq, n_pos):
        """float32 [n_pos, hd/2, 2] = (cos, sin)(float(p) * inv_freq[k]), computed on the device."""
        t = native.torch()
        table = t.empty((n_pos, inv_freq.shape[0], 2), dtype=t.float32, device=inv_freq.device)
        self._call("rope_table", [inv_freq, table])
        return table

    def qk_norm_rope_kv_write(self, qkv, q_w, k_w, eps, inv_freq, positions, slots, view, pool, q_out, heads, kv_heads,
                              head_dim, rope_table=None):
        """qkv f32 [M, (heads + 2 kv_heads) hd] -> q_out T [M, heads hd] and the cache pages.
        kv_heads = 0: only q (nothing is written to the cache)."""
        self._call("qk_norm_rope_kv_write", [qkv, q_w, k_w, inv_freq, rope_table, positions, slots, view.table, pool, q_out],
                   [eps, heads, kv_heads, head_dim], fold=(8,))

    def qk_norm_inplace(self, qkv, q_w, k_w, eps, heads, kv_heads, head_dim):
        self._call("qk_norm_inplace", [qkv, q_w, k_w], [eps, heads, kv_heads, head_dim])

    def can_fuse_norm(self, n_rows: int, dtype) -> bool:
        """Whether `linear` has a kernel that takes the norm of this many rows in."""
        return bool(self._call("can_fuse_norm", [], [n_rows, native.dtype_code(dtype)], libs=["core"]))

    def linear(self, a, w, out, epilogue: str, may_defer: bool = False):
        """out (op)= a w^T.  a: T [M, K] (rows may be strided); w: T [N, K] contiguous.
        epilogue: "store" f32 out = ; "add" f32 out += ; "store_act" T out = ;
        "swiglu": w is [2F, K] = [gate; up], T out [M, F] = silu(gate) * up.
        may_defer (with "add"): the caller reads `out` next through this object (see `flush`)."""
        libs = ["gemm_generic"] + (["gemm_bf16", "core"] if w.dtype == native.torch().bfloat16 and self.use_fast_gemm else [])
        if isinstance(a, NormedRows):
            self._call("linear_normed", [a.x, a.weight, a.out, w, out], [a.eps, EPI[epilogue], int(may_defer)],
                       libs=libs + ["core"])
        else:
            self._call("linear", [a, w, out], [EPI[epilogue], int(may_defer)], libs=libs)

    def _linear_normed(self, a: NormedRows, w, out, epilogue: str) -> bool:
        """rmsnorm and product in one kernel; False if no kernel serves the shape (nothing was launched)."""
        return bool(self._call("linear_normed_only", [a.x, a.weight, a.out, w, out], [a.eps, EPI[epilogue]],
                               libs=["gemm_bf16", "core"]))

    def qkv_prepared(self, a, w, q_w, k_w, eps, inv_freq, rope_table, positions, slots, view, pool, q_out, heads, kv_heads,
                     head_dim) -> bool:
        """`linear(a, w, qkv, "store")` and `qk_norm_rope_kv_write` in one kernel, for steps of many tokens
        in bfloat16.  False if no kernel serves the step (nothing has been done then)."""
        if isinstance(a, NormedRows):
            return False
        return bool(self._call("qkv_prepared", [a, w, q_w, k_w, inv_freq, rope_table, positions, slots, view.table, pool, q_out],
                               [eps, heads, kv_heads, head_dim], fold=(9,), libs=["gemm_bf16", "core"]))

    # ----------------------------------------------------------------- attention
    def attention_rows(self, q, pool, table, positions, slots, out, heads, kv_heads, head_dim, scale, window):
        self._call("attention_rows", [q, pool, table, positions, slots, out], [heads, kv_heads, head_dim, scale, int(window or 0)],
                   fold=(1,))

    @staticmethod
    def _work(ctx):
        """The attention's work lists as a step context (or a test's stand-in for one) holds them."""
        g = lambda n, d=None: getattr(ctx, n, d)
        tensors = [ctx.positions, ctx.slots, g("entry_meta"), g("tiles"), g("tiles_small"), g("decode_rows")]
        numbers = [ctx.M, g("n_tiles", 0), g("n_tiles_small", 0), g("n_decode_rows", 0), int(bool(ctx.decode_only)),
                   g("max_context", 0), g("portion_context", 0), g("split_context", g("max_context", 0))]
        return tensors, numbers

    def attention(self, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window, softcap: float = 0.0):
        """Attention of every row of the step over its request's pages.  softcap > 0: scores are capped,
        s <- softcap tanh(s / softcap), before the softmax."""
        t, n = self._work(ctx)
        libs = ["attention_generic"] + (["attention_bf16"] if q.dtype == native.torch().bfloat16 and self.use_fast_attention else [])
        rows_are_slots = bool(getattr(ctx, "slots_are_rows", False))
        rows = [0.0, 0, int(rows_are_slots), float(softcap)] if rows_are_slots or softcap else []   # (unused, unused, slots[m] == m, cap)
        self._call("attention", [q, pool, view.table, out] + t, [heads, kv_heads, head_dim, scale, int(window or 0)] + n + rows,
                   fold=(1,), libs=libs)

    def attention_from_projections(self, ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool, write_kv, out, heads,
                                   kv_heads, head_dim, scale, window) -> bool:
        """`qk_norm_rope_kv_write` and `attention` in one kernel, for steps of single tokens in bfloat16.
        False if no kernel serves the step (nothing has been done then)."""
        if not self.use_fast_attention:
            return False
        t, n = self._work(ctx)
        return bool(self._call("attention_from_projections", [qkv, pool, view.table, out] + t + [q_w, k_w, inv_freq, rope_table],
                               [heads, kv_heads, head_dim, scale, int(window or 0)] + n + [eps, int(bool(write_kv))] +
                               ([1] if getattr(ctx, "slots_are_rows", False) else []),
                               fold=(1,), libs=["attention_bf16", "core"]))

    # ------------------------------------------------------------------ sampling
    # ---- layers beyond the pre-norm transformer block
    def add_sinusoid(self, x, positions, inv_freq):
        """x f32 [M, H]: x[m, 2i] += sin(pos[m] inv_freq[i]), x[m, 2i + 1] += cos(the same)."""
        self._call("add_sinusoid", [x, positions, inv_freq])

    def add_row(self, x, v):
        self._call("add_row", [x, v])

    def xielu(self, z, act, out):
        """out = xIELU(z) with act = (p, q), z float32."""
        self._call("xielu", [z, act, out])

    def scaled_add(self, x, a, sa=None, b=None, sb=None):
        """x += a * sa + b * sb per channel."""
        self._call("scaled_add", [x, a, sa, b, sb])

    def qkv_split_write(self, qkv, positions, slots, table, pool, q_out, heads, kv_heads, dk, dv, coef=0.0, every=1):
        """qkv f32 [M, heads dk + kv_heads (dk + dv)]; pool [pages, kv_heads, P, dk + dv] (a page: K [kv][P][dk] | V [kv][dv][P])."""
        self._call("qkv_split_write", [qkv, positions, slots, table, pool, q_out], [heads, kv_heads, dk, dv, coef, every])

    def attention_capped(self, q, pool, table, positions, slots, out, heads, kv_heads, dk, dv, scale, softcap=0.0, window=0):
        self._call("attention_capped", [q, pool, table, positions, slots, out],
                   [heads, kv_heads, dk, dv, scale, softcap, int(window or 0)])

    def mlstm_scan(self, proj, bias_i, bias_f, state, entries, o, heads, dk, dv, cap, q_scale, columns, chunks=None, spans=None):
        """entries int32 [R, 4] = (first row, tokens, -, state slot); columns = (q, k, v, i, f) of proj.  chunks int32
        [n, 4] = (entry, first row, tokens, 1: the entry's first chunk + 2: its last) and spans int32 [R, 2] = (first
        chunk, chunks): the entries' tokens run as chunks side by side."""
        self._call("mlstm_scan", [proj, bias_i, bias_f, state, entries, o, chunks, spans], [heads, dk, dv, cap, q_scale] + list(columns))

    def gated_head_norm(self, o, proj, gate_col, w, eps, out, heads, dv):
        self._call("gated_head_norm", [o, proj, w, out], [gate_col, eps, heads, dv])

    # ---- post-norm layers, short convolutions, differential attention, mixtures of experts
    def norm_residual(self, x, y, gain, eps, accumulate=True, gather=None, rounded=None):
        """x (+)= y / rms(y) * gain, all float32; gather int32 [M, n]: row m of y is the sum of the rows y[gather[m, k]];
        rounded: also receives the new x in its own dtype."""
        self._call("norm_residual", [x, y, gain, gather, rounded], [eps, int(bool(accumulate))])

    def round_rows(self, x, out):
        self._call("round_rows", [x, out])

    def scale(self, x, s):
        self._call("scale", [x], [s])

    def short_conv(self, u, taps, state, entries, entry_of, positions, out):
        """out[m, c] = sum_j taps[c, j] u(pos[m] - (K - 1) + j)[c]; state f32 [slots, K - 1, C] holds the rows before each
        entry's start and is left with the last K - 1 rows; entries int32 [R, 4] = (first row, tokens, start, slot)."""
        self._call("short_conv", [u, taps, state, entries, entry_of, positions, out])

    def diff_qk_prep(self, qkv, q_w, k_w, inv_freq, rope_table, positions, slots, table, pool, q_out, eps, heads, kv_heads, dk, dv,
                     rot_dims=0, mag=1.0, taps=None, state=None, entries=None):
        """qkv f32 [M, heads 2 dk + kv_heads (2 dk + dv)]; pool [pages, kv_heads, P, 2 dk + dv] (K [kv][P][2 dk] | V [kv][dv][P]).
        taps f32 [C, K] with state f32 [slots, K - 1, C] and entries int32 [R, 4] (slots names every row's entry): the short
        convolution of `short_conv` on every channel first, inside the same kernel."""
        tensors = [qkv, q_w, k_w, inv_freq, rope_table, positions, slots, table, pool, q_out]
        if taps is not None:
            tensors += [taps, state, entries]
        self._call("diff_qk_prep", tensors, [eps, heads, kv_heads, dk, dv, rot_dims, mag])

    def diff_attention(self, q, pool, table, positions, slots, out, heads, kv_heads, dk, dv, scale, lam, eps, out_scale, block=0, window=0,
                       tiles=None, rows=None, entries=None, all_rows=False, context=0):
        """tiles int32 [n, 3] = (entry, first row, rows <= 64) with entries int32 [R, 4] = (row0, tokens, start, -), rows int32 [n]
        (or all_rows: every row is a single token): the lists of the bfloat16 matrix-core kernels; without them every row is
        walked on its own."""
        tensors, numbers = [q, pool, table, positions, slots, out], [heads, kv_heads, dk, dv, scale, int(block or 0), int(window or 0), lam, eps, out_scale]
        libs = ["diff_attention"]
        if tiles is not None or rows is not None or all_rows:
            tensors += [tiles, rows, entries]
            numbers.append(q.shape[0] if all_rows else 0)
            if context:
                numbers.append(context)        # the longest context of a single row: its keys may be split over workgroups
            if q.dtype == native.torch().bfloat16:
                libs.append("diff_attention_bf16")
        self._call("diff_attention", tensors, numbers, libs=libs)

    def moe_route(self, h, router, ids, wts, top, score="sigmoid", renormalize=False):
        """score "softmax_chosen": the largest logits are chosen and the weights are the softmax over the chosen logits alone."""
        self._call("moe_route", [h, router, ids, wts], [top, {"sigmoid": 0, "softmax": 1, "softmax_chosen": 2}[score], int(bool(renormalize))])

    def moe_experts_gated(self, h, ids, wts, gate_up, down, y, experts, activation="clamped", limit=0.0, alpha=1.702):
        """y f32 [M, W] = sum_k s_k down_e act(gate_e h, up_e h); gate_up [experts 2F, W] holds an expert's gate rows above its up rows."""
        libs = ["moe"] + (["moe_bf16"] if h.dtype == native.torch().bfloat16 else [])
        self._call("moe_experts_gated", [h, ids, wts, gate_up, down, y], [experts, {"silu": 0, "clamped": 1}[activation], limit, alpha], libs=libs)

    # ---- Dynamic Tanh, gated activations, biased and partly rotated q/k/v, latent attention
    def dyt(self, x, alpha, w, b, out, rows=None):
        """out[r] = tanh(alpha x[rows[r] or r]) * w + b; x float32, alpha float32 [1]."""
        self._call("dyt", [x, alpha, w, b, out, rows])

    def gated_act(self, z, bias, out, activation="silu", limit=0.0, alpha=1.702):
        """z f32 [R, 2F] = [gate | up] (+ bias [2F]); "silu": silu(g) u; "clamped": g = min(g, limit), u = clamp(u, +-limit),
        g sigmoid(alpha g) (u + 1)."""
        self._call("gated_act", [z, bias, out], [{"silu": 0, "clamped": 1, "gelu_tanh": 2}[activation], limit, alpha])

    # ---- the layer norm, a residual in several streams, gated attention, linear attention with a fixed decay, a grouped router
    def layernorm(self, x, w, eps, out, rows=None):
        """out[r] = (x - mean) / sqrt(var + eps) * w of row rows[r] (or r); x float32; out may be x."""
        self._call("layernorm", [x, w, out, rows], [eps])

    def layernorm_mixed(self, streams, coef, w, eps, out):
        """The same of sum_s coef[s] streams[s]; streams float32 [S, M, H]."""
        self._call("layernorm_mixed", [streams, coef, w, out], [eps])

    def hyper_combine(self, streams, coef, u):
        self._call("hyper_combine", [streams, coef, u])

    def hyper_spread(self, x, streams):
        self._call("hyper_spread", [x, streams])

    def hyper_write(self, streams, mix, back, y, y2=None, f1=1.0, f2=1.0, next_coef=None, next_w=None, eps=0.0, next_out=None):
        """streams[t] <- sum_s mix[s, t] streams[s] + back[t] y, every t at once; with y2 the output is f1 y + f2 y2; with next_*
        the same pass leaves next_out = layernorm(sum_t next_coef[t] streams[t]) * next_w of the new streams."""
        self._call("hyper_write", [streams, mix, back, y, y2, next_coef, next_w, next_out], [f1, f2, eps])

    def gated_qkv_prep(self, proj, q_w, k_w, inv_freq, rope_table, positions, slots, table, pool, q_out, heads, kv_heads, dk, dv, columns,
                       eps=1e-6, rot_dims=0, mix_mode=0, mix_lambda=None, kept=None):
        """proj f32 [M, N] with q, k, v from `columns` on (v < 0: the values are the keys as projected); per-head norms (q_w, k_w
        or None), rotation of the first rot_dims entries, mix_mode 1: the values also go to `kept`; 2: v <- (1 - l) v + l kept."""
        self._call("gated_qkv_prep", [proj, q_w, k_w, inv_freq, rope_table, positions, slots, table, pool, q_out, mix_lambda, kept],
                   [eps, heads, kv_heads, dk, dv] + list(columns) + [rot_dims, mix_mode])

    def gated_attention(self, q, pool, table, positions, slots, sink, gate_proj, out, heads, kv_heads, dk, dv, scale, window=0, gate_col=0,
                        gate_mode=0):
        """Causal softmax attention with exp(sink[h]) in the denominator (sink None: none) and the output times sigmoid of the
        gate columns of gate_proj (gate_mode 1: one an entry, 2: one a head, 0: none)."""
        self._call("gated_attention", [q, pool, table, positions, slots, sink, gate_proj, out],
                   [heads, kv_heads, dk, dv, scale, int(window or 0), gate_col, gate_mode])

    def decay_scan(self, proj, decay, state, entries, o, heads, dk, dv, columns, chunks=None, spans=None):
        """entries int32 [R, 4] = (first row, tokens, -, state slot); S <- decay S + k v^T, o = S^T q on silu'd columns of proj.
        chunks int32 [n, 4] = (entry, first row, tokens, 1: the entry's first chunk + 2: its last) and spans int32 [R, 2] = (first
        chunk, chunks): the entries' tokens run as chunks side by side."""
        self._call("decay_scan", [proj, decay, state, entries, o, chunks, spans], [heads, dk, dv] + list(columns))

    def gated_row_norm(self, o, proj, gate_col, w, eps, out):
        self._call("gated_row_norm", [o, proj, w, out], [gate_col, eps])

    def moe_route_grouped(self, h, router, ids, wts, correction, top, groups=0, keep=0, weight_scale=1.0, sum_floor=0.0, renormalize=True):
        """Sigmoid scores; `correction` joins them for the choice only; only experts of the `keep` best of `groups` groups can be chosen."""
        self._call("moe_route_grouped", [h, router, ids, wts, correction], [top, 0, int(bool(renormalize)), groups, keep, weight_scale, sum_floor])

    def concat_round(self, a, b, out):
        self._call("concat_round", [a, b, out])

    def qkv_prep_write(self, qkv, bias, inv_freq, rope_table, positions, slots, table, pool, q_out, heads, kv_heads, dk, dv,
                       rot_dims=0, mag=1.0, coef=0.0, every=1):
        """`qkv_split_write` with a bias on every column first and the rotation of the first rot_dims entries of every query and key head."""
        self._call("qkv_prep_write", [qkv, bias, inv_freq, rope_table, positions, slots, table, pool, q_out],
                   [heads, kv_heads, dk, dv, coef, every, rot_dims, mag])

    def latent_prep(self, proj, norm_w, inv_freq, rope_table, positions, slots, table, pool, off_kv, eps, heads, dim, rot_dim, rank,
                    rot_dims=0, mag=1.0):
        """proj f32 [M, >= off_kv + rank + rot_dim]: the latent normed and the shared key part rotated into pool [pages, P, rank + rot_dim];
        the heads' rotated query parts turned in place."""
        self._call("latent_prep", [proj, norm_w, inv_freq, rope_table, positions, slots, table, pool],
                   [off_kv, eps, heads, dim, rot_dim, rank, rot_dims, mag])

    def latent_attention(self, proj, w_uk, w_uv, sink, pool, table, positions, slots, out, heads, dim, rot_dim, rank, v_dim, scale, window=0,
                         w_uk_t=None, tiles=None, rows=None, entries=None, all_rows=False, context=0):
        """pool [pages, P, rank + rot_dim], or [pages, P, 2 rank + rot_dim] (a page: its P rows, then the latents transposed
        [rank][P]).  w_uk_t (`latent_transpose` of w_uk) with tiles int32 [n, 3] = (entry, first row, rows <= 64) and entries
        int32 [R, 4] = (row0, tokens, start, -), rows int32 [n] (or all_rows: every row is a single token): the bfloat16
        matrix-core kernels; without them every row is walked on its own."""
        tensors, numbers = [proj, w_uk, w_uv, sink, pool, table, positions, slots, out], [heads, dim, rot_dim, rank, v_dim, scale, int(window or 0)]
        libs = ["latent_attention"]
        if w_uk_t is not None:
            tensors += [w_uk_t, tiles, rows, entries]
            numbers += [proj.shape[0] if all_rows else 0, int(context or 0)]
            if out.dtype == native.torch().bfloat16:
                libs.append("latent_attention_bf16")
        self._call("latent_attention", tensors, numbers, libs=libs)

    def latent_transpose(self, src, dst, heads):
        """dst [heads cols, rows] = src [heads rows, cols], every head's matrix transposed."""
        self._call("latent_transpose", [src, dst], [heads])

    def moe_experts(self, h, ids, wts, up, down, y, experts, scale_input=True):
        """y f32 [M, W] = sum over a token's experts; up [experts F, W], down [experts W, F]."""
        libs = ["moe"] + (["moe_bf16"] if h.dtype == native.torch().bfloat16 else [])
        self._call("moe_experts", [h, ids, wts, up, down, y], [experts, int(bool(scale_input))], libs=libs)

    def argmax(self, logits, out):
        if out.dtype != native.torch().int32 or out.shape[0] < logits.shape[0]:
            raise KernelError("argmax: logits must be contiguous float32 [n, V], out int32 [n]")
        self._call("argmax", [logits, out])

    def sample(self, logits, temperature, top_k, top_p, uniform, out):
        t = native.torch()
        n = logits.shape[0]
        for x, dt in ((temperature, t.float32), (top_k, t.int32), (top_p, t.float32), (uniform, t.float32), (out, t.int32)):
            if x.dtype != dt or x.shape[0] < n:
                raise KernelError("sample: per-row arguments must be float32/int32 [n]")
        self._call("sample", [logits, temperature, top_k, top_p, uniform, out])


# ---------------------------------------------- how the host library hands rows to the attention kernels
SERVED_HEAD_DIMS = (32, 64, 128)     # head sizes of the bfloat16 matrix-core attention kernels
MAX_SPLITS = 64                      # the merge kernel's limit
MIN_BLOCKS_PER_SPLIT = 16            # four 16-key blocks per wavefront at least


def compute_units() -> int:
    return int(get_ops()._call("compute_units", libs=["core"]))


def decode_splits(n_rows: int, kv_heads: int, heads: int, context: int, typical: int = 0, head_dim: int = 128) -> int:
    """Into how many runs the decode kernel splits the context (`Ops::decode_splits`, ops/ops.cpp)."""
    return int(native.lib().ti_decode_splits(n_rows, kv_heads, heads, context, typical or context, compute_units(), head_dim))


def portion_launch(ctx, heads: int, window: int):
    """(runs of keys, paired) for the prefill kernel with 64-row tiles (`Ops::portion_launch`)."""
    paired = ctypes.c_int()
    runs = native.lib().ti_portion_launch(ctx.n_tiles_small, heads, getattr(ctx, "portion_context", 0), int(window or 0),
                                          compute_units(), ctypes.byref(paired))
    return int(runs), bool(paired.value)


_OPS: Optional[Ops] = None


def get_ops() -> Ops:
    """An `Ops` object of the process for code that runs kernels outside an engine."""
    global _OPS
    if _OPS is None:
        _OPS = Ops()
    return _OPS
