"""Prefill and decode throughput of the Fasovik design at layer sizes of real models (random weights), beside the engine's closest GGUF model — a Llama-architecture model of the
same width, depth and head count with Q8_0 weights, the densest quantised type the mat-vec kernels take — and the kernels' distance from the roofline for both.

`bench.py --compare-hybrid [SIZE,...]` prints one JSON line per size; bench.py's default workload and line are untouched.

`bench.py --compare-parallel [SIZE,...]` does the same for the Vikarax design (parallel mixer: chunked sigmoid attention beside a selective recurrence, gated experts with a
shared one) beside the engine's closest model, which is Fasovik at the same width, depth, head sizes and expert sizes.

`bench.py --compare-postnorm [SIZE,...]`: the Rafusun design (delta-rule layers and attention + time-mix layers in turn, a gated dense feed-forward, the norm after the sum) beside the
closest model, which is Vikarax at the same width, depth, attention sizes and with a dense feed-forward of the same width.

`bench.py --compare-window [SIZE,...]`: the Rarevik design (one tanh norm per layer, sliding-window attention with pooled far blocks and a sink or with a head gate, clipped routed experts with a
gated shared one, a repeated run's input matrix) beside the closest model, which is Vikarax at the same width, depth, attention and expert sizes."""
import ctypes as C
import json
import os
import struct
import sys
import time

import numpy as np

from .. import lib as L, llama as LL
from . import synth

HBM_PEAK = 8.0e12
BF16_PEAK = 2.5e15

# name -> width, layers, heads, dim, vdim, kv_rank, experts, identity, top, ff, vocab
SIZES = {
    "w1024": (1024, 4, 16, 64, 64, 256, 8, 2, 2, 512, 32000),
    "w2048": (2048, 4, 16, 128, 128, 512, 8, 2, 2, 1024, 32000),
    "w4096": (4096, 2, 32, 128, 128, 512, 8, 2, 2, 2048, 32000),
}
FAMILIES = {0: "matvec", 1: "matrix_cores", 2: "norm_quant", 3: "quant", 4: "act_quant", 5: "attention", 6: "other"}


def write_fasovik(folder, size, seed=1):
    width, n_layer, heads, dim, vdim, rank, n_exp, n_id, top, ff, vocab = SIZES[size]
    layers = []
    for i in range(n_layer):
        mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n_exp, "identity": n_id, "top": top}}
        if i % 2 == 0:
            layers.append({"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": dim ** -0.5}, "mlp": mlp})
        else:
            layers.append({"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": [float(1.0 - 2.0 ** (-3 - 5 * h / heads)) for h in range(heads)]}, "mlp": mlp})
    cfg = {"architecture": "Fasovik", "vocab": vocab, "width": width, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5}, "residual_mult": 0.5, "layers": layers}
    shapes = {"embed": (vocab, width), "final.norm": (width,)}
    for i, l in enumerate(layers):
        p = "l%d." % i
        shapes[p + "norm1"] = shapes[p + "norm2"] = (width,)
        hd, hv = heads * dim, heads * vdim
        if l["type"] == "lightning":
            shapes.update({p + "mix.q": (hd, width), p + "mix.k": (hd, width), p + "mix.v": (hv, width), p + "mix.g": (hv, width), p + "mix.o": (width, hv), p + "mix.norm": (hv,)})
        else:
            shapes.update({p + "mix.q": (hd, width), p + "mix.dkv": (rank, width), p + "mix.dkv.norm": (rank,), p + "mix.uk": (hd, rank), p + "mix.uv": (hv, rank), p + "mix.sink": (heads,), p + "mix.o": (width, hv)})
        shapes[p + "mlp.router"] = (n_exp + n_id, width)
        shapes[p + "mlp.correction"] = (n_exp + n_id,)
        for e in range(n_exp):
            shapes[p + "mlp.e%d.up" % e] = (ff, width)
            shapes[p + "mlp.e%d.down" % e] = (width, ff)
    os.makedirs(folder, exist_ok=True)
    head, at = {}, 0
    for name, shp in shapes.items():
        n = int(np.prod(shp)) * 2
        head[name] = {"dtype": "BF16", "shape": list(shp), "data_offsets": [at, at + n]}
        at += n
    h = json.dumps(head).encode()
    h += b" " * (-len(h) % 8)
    rng = np.random.default_rng(seed)
    with open(os.path.join(folder, "model.safetensors.part"), "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h)
        for name, shp in shapes.items():
            if len(shp) == 1:
                v = rng.standard_normal(shp, dtype=np.float32) * 0.1 + (1.0 if name.endswith("mix.norm") or name.endswith("dkv.norm") else 0.0)
            else:
                v = rng.standard_normal(shp, dtype=np.float32) * np.float32(shp[-1] ** -0.5)
            f.write((v.view(np.uint32) >> 16).astype(np.uint16).tobytes())
    os.replace(os.path.join(folder, "model.safetensors.part"), os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return folder


# Vikarax at the sizes above: name -> key/value heads, rotated dimensions, chunk, recurrence heads x vdim, state, groups, router groups (count, keep), shared expert's ff
VIKARAX = {
    "w1024": (4, 32, 256, 16, 64, 64, 2, 2, 1, 512),
    "w2048": (4, 64, 256, 32, 64, 128, 2, 2, 1, 1024),
    "w4096": (8, 64, 512, 64, 64, 128, 4, 4, 2, 2048),
}


def write_random_tensors(folder, cfg, shapes, ones=(), seed=1):
    """a model folder of random bfloat16 tensors: vectors around 0 (around 1 where the name ends in one of `ones`), matrices of unit row norm"""
    os.makedirs(folder, exist_ok=True)
    head, at = {}, 0
    for name, shp in shapes.items():
        n = int(np.prod(shp)) * 2
        head[name] = {"dtype": "BF16", "shape": list(shp), "data_offsets": [at, at + n]}
        at += n
    h = json.dumps(head).encode()
    h += b" " * (-len(h) % 8)
    rng = np.random.default_rng(seed)
    with open(os.path.join(folder, "model.safetensors.part"), "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h)
        for name, shp in shapes.items():
            if len(shp) == 0:
                v = np.full((), 0.5, np.float32)
            elif len(shp) == 1 or name.endswith(".conv"):
                v = rng.standard_normal(shp, dtype=np.float32) * 0.1 + (1.0 if name.endswith(tuple(ones)) else 0.0)
            else:
                v = rng.standard_normal(shp, dtype=np.float32) * np.float32(shp[-1] ** -0.5)
            f.write((v.view(np.uint32) >> 16).astype(np.uint16).tobytes())
    os.replace(os.path.join(folder, "model.safetensors.part"), os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    return folder


def write_vikarax(folder, size, seed=1, dense_ff=0):
    """dense_ff > 0: a dense feed-forward of that width in place of the routed experts"""
    width, n_layer, heads, dim, vdim, _, n_exp, _, top, ff, vocab = SIZES[size]
    kv_heads, rot, chunk, r_heads, r_vdim, state, groups, g_count, g_keep, shared = VIKARAX[size]
    inner, gn = r_heads * r_vdim, groups * state
    layers, shapes = [], {"embed": (vocab, width), "head": (vocab, width), "final.norm": (width,), "final.norm.b": (width,)}
    for i in range(n_layer):
        mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n_exp, "top": top, "groups": {"count": g_count, "keep": g_keep}}, "shared": {"ff": shared}}
        left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "rot": {"dims": rot, "base": 10000.0}, "mask": {"size": chunk}}
        right = {"heads": r_heads, "vdim": r_vdim, "state": state, "groups": groups, "conv": 4, "norm_groups": groups}
        if dense_ff:
            mlp = {"kind": "dense", "ff": dense_ff}
        layers.append({"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": 0.7, "right_scale": 0.7}, "mlp": mlp})
        p = "l%d." % i
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            shapes[p + n] = shapes[p + n + ".b"] = (width,)
        shapes[p + "dwa"] = (i + 2,)
        q = p + "mix.left."
        shapes.update({q + "q": (heads * dim, width), q + "k": (kv_heads * dim, width), q + "v": (kv_heads * vdim, width), q + "q.norm": (dim,), q + "k.norm": (dim,), q + "pb": (heads,),
                       q + "g": (heads, width), q + "o": (width, heads * vdim)})
        q = p + "mix.right."
        shapes.update({q + "in": (2 * inner + 2 * gn + r_heads, width), q + "conv": (inner + 2 * gn, 4), q + "conv.b": (inner + 2 * gn,), q + "dt_bias": (r_heads,), q + "A_log": (r_heads,),
                       q + "D": (r_heads,), q + "norm": (inner,), q + "o": (width, inner)})
        if dense_ff:
            shapes.update({p + "mlp.up": (dense_ff, width), p + "mlp.down": (width, dense_ff)})
            continue
        shapes[p + "mlp.router"] = (n_exp, width)
        for e in ["e%d" % e for e in range(n_exp)] + ["shared"]:
            f = shared if e == "shared" else ff
            shapes.update({p + "mlp.%s.gate" % e: (f, width), p + "mlp.%s.up" % e: (f, width), p + "mlp.%s.down" % e: (width, f)})
    cfg = {"architecture": "Vikarax", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "logit_softcap": 30.0, "layers": layers}
    return write_random_tensors(folder, cfg, shapes, ones=("norm", "norm1", "norm2", "norm1b", "norm2b", "dwa", ".D"), seed=seed)


def write_rafusun(folder, size, seed=1):
    """layers in turn: a delta-rule mixer without a feed-forward, then attention + time mixing with a gated dense feed-forward (attention sizes as the Vikarax model of this size)"""
    width, n_layer, heads, dim, vdim, _, _, _, _, ff, vocab = SIZES[size]
    kv_heads, rot, chunk, r_heads, r_vdim, _, _, _, _, _ = VIKARAX[size]
    dense_ff, rank = 4 * ff, 64
    layers, shapes = [], {"embed": (vocab, width), "bigram": (65537, width), "head": (vocab, width), "final.norm": (width,)}
    for i in range(n_layer):
        p = "l%d." % i
        shapes[p + "norm1"] = shapes[p + "ls1"] = (width,)
        if i % 2 == 0:
            layers.append({"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": 4}, "mlp": None})
            q = p + "mix."
            shapes.update({q + "q": (kv_heads * dim, width), q + "k": (kv_heads * dim, width), q + "v": (heads * vdim, width), q + "q.conv": (kv_heads * dim, 4), q + "k.conv": (kv_heads * dim, 4),
                           q + "v.conv": (heads * vdim, 4), q + "b": (heads, width), q + "A_log": (heads,), q + "dt_bias": (heads * dim,), q + "a1": (rank, width), q + "a2": (heads * dim, rank),
                           q + "g1": (rank, width), q + "g2": (heads * vdim, rank), q + "norm": (vdim,), q + "o": (width, heads * vdim)})
            continue
        left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "softcap": 30.0, "rot": {"dims": rot, "base": 10000.0}, "mask": {"size": chunk}}
        layers.append({"type": "parallel", "mixer": {"left": left, "right": {"heads": r_heads, "dim": r_vdim}}, "mlp": {"kind": "dense", "ff": dense_ff}})
        inner = r_heads * r_vdim
        q = p + "mix.left."
        shapes.update({q + "q": (heads * dim, width), q + "k": (kv_heads * dim, width), q + "v": (kv_heads * vdim, width), q + "o": (width, heads * vdim), q + "out": (width,)})
        q = p + "mix.right."
        shapes.update({q + "mu." + n: (width,) for n in "rkvgw"})
        shapes.update({q + n: (inner, width) for n in "rkvg"})
        shapes.update({q + "w1": (rank, width), q + "w2": (inner, rank), q + "w0": (inner,), q + "u": (r_heads, r_vdim), q + "norm": (inner,), q + "o": (width, inner), q + "out": (width,)})
        shapes.update({p + "norm2": (width,), p + "ls2": (width,), p + "mlp.gate": (dense_ff, width), p + "mlp.up": (dense_ff, width), p + "mlp.down": (width, dense_ff)})
    cfg = {"architecture": "Rafusun", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "postln_alpha": 2.0, "embedding": {"scale": 1.0, "bigram": {"buckets": 65536, "mul_prev": 8191, "mul_cur": 31}},
           "layers": layers}
    return write_random_tensors(folder, cfg, shapes, ones=("norm", "norm1", "norm2", "ls1", "ls2", ".out"), seed=seed)


# Rarevik at the sizes above: pooled block, convolution taps (attention sizes, window = the Vikarax model's chunk, expert sizes as the Vikarax model of the size)
RAREVIK = {"w1024": (16, 4), "w2048": (16, 4), "w4096": (32, 4)}


def write_rarevik(folder, size, seed=1):
    """layers in turn: window attention with a convolution, pooled far blocks and a sink, then window attention with stretched rotation steps and a head gate; every layer with routed clipped experts
    and a gated shared one; layers 1 .. 2 are a (once-run) repeated run, so the run's input matrix is part of a pass"""
    width, n_layer, heads, dim, vdim, _, n_exp, _, top, ff, vocab = SIZES[size]
    kv_heads, rot, chunk, _, _, _, _, _, _, shared = VIKARAX[size]
    pool, conv = RAREVIK[size]
    layers, shapes = [], {"embed": (vocab, width), "loop.in": (width, 2 * width), "final.norm": (width,), "final.norm.b": (width,), "final.norm.alpha": ()}
    for i in range(n_layer):
        p, q = "l%d." % i, "l%d.mix." % i
        mlp = {"kind": "moe", "expert": {"ff": ff, "limit": 7.0}, "router": {"experts": n_exp, "top": top}, "shared": {"ff": shared, "limit": 7.0}}
        mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "rot": {"dims": rot, "base": 10000.0}, "mask": {"size": chunk}}
        shapes.update({p + "norm1": (width,), p + "norm1.b": (width,), p + "norm1.alpha": (), p + "shift": (width,),
                       q + "q": (heads * dim, width), q + "k": (kv_heads * dim, width), q + "v": (kv_heads * vdim, width), q + "o": (width, heads * vdim)})
        if i % 2 == 0:
            mx["conv"] = conv
            mx["mask"]["pool"] = pool
            shapes.update({q + "q.conv": (heads * dim, conv), q + "k.conv": (kv_heads * dim, conv), q + "v.conv": (kv_heads * vdim, conv), q + "q.norm": (dim,), q + "k.norm": (dim,), q + "sink": (heads,)})
        else:
            mx["rot"]["scaling"] = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}
            shapes[q + "g"] = (heads, width)
        layers.append({"type": "attention" if i % 2 == 0 else "attention_2", "mixer": mx, "mlp": mlp})
        shapes.update({p + "mlp.router": (n_exp, width), p + "mlp.router.b": (n_exp,), p + "mlp.shared.sg": (1, width)})
        for e in ["e%d" % e for e in range(n_exp)] + ["shared"]:
            f = shared if e == "shared" else ff
            shapes.update({p + "mlp.%s.gate" % e: (f, width), p + "mlp.%s.up" % e: (f, width), p + "mlp.%s.down" % e: (width, f)})
    cfg = {"architecture": "Rarevik", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": min(3, n_layer), "times": 1}, "layers": layers}
    return write_random_tensors(folder, cfg, shapes, ones=("norm", "norm1"), seed=seed)


class KtRow(C.Structure):          # struct pi_kt_row (include/pipeinfer_ops.h)
    _fields_ = [("family", C.c_int32), ("type", C.c_int32), ("n_tok", C.c_int32), ("sampled_dropped", C.c_int32), ("shape_bytes", C.c_uint64), ("launches", C.c_uint64),
                ("bytes_total", C.c_double), ("sampled", C.c_uint64), ("avg_us", C.c_double), ("avg_sampled_bytes", C.c_double)]


def kernel_table(lib, fn):
    """runs fn() with every eager launch timed; -> {family: {launches, us, bytes, hbm_frac}}"""
    lib.pi_kernel_timing(1, 1)
    fn()
    L.check(lib.pi_device_sync())
    buf = (KtRow * 4096)()
    n = lib.pi_kernel_timing_rows(buf, 4096)
    lib.pi_kernel_timing(0, 1)
    out = {}
    for r in buf[:n]:
        f = out.setdefault(FAMILIES.get(r.family, "other"), {"launches": 0, "us": 0.0, "bytes": 0.0})
        f["launches"] += int(r.launches)
        f["us"] += float(r.avg_us) * int(r.launches)
        f["bytes"] += float(r.bytes_total)
    for f in out.values():
        f["hbm_frac"] = round(f["bytes"] / (f["us"] * 1e-6) / HBM_PEAK, 4) if f["us"] > 0 else None
        f["us"] = round(f["us"], 1); f["bytes"] = int(f["bytes"])
    return out


def measure(lib, path, n_prompt, n_decode, hybrid, exact=False):
    model = LL.Model(path)
    ctx = LL.Context(model, n_ctx=n_prompt + n_decode + 64, n_batch=n_prompt)
    if hybrid:
        ctx.set_precision(exact)
    rng = np.random.default_rng(7)
    toks = [int(t) for t in rng.integers(1, model.n_vocab, n_prompt + n_decode)]
    res = {}
    ctx.feed(toks[:n_prompt], 0, 0)                              # warm-up: upload, graph capture
    ctx.feed(toks[n_prompt:n_prompt + 2], n_prompt, 0)
    ctx.seq_rm(0, -1, -1)
    t_pre = []
    ctx.reset_stats()
    for _ in range(3):
        L.check(lib.pi_device_sync()); t0 = time.perf_counter()
        ctx.feed(toks[:n_prompt], 0, 0)
        t_pre.append(time.perf_counter() - t0)
        if _ < 2:
            ctx.seq_rm(0, -1, -1)
    st = ctx.stats()
    res["prefill_gpu_ms"] = round(st["gpu_ms"] / max(1, st["n_calls"]), 3)       # the pass on the GPU (graph replay + the logits' way to the host), without this script's copies
    ctx.reset_stats()
    t0 = time.perf_counter()
    for i in range(n_decode):
        ctx.feed(toks[n_prompt + i:n_prompt + i + 1], n_prompt + i, 0)
    t_dec = time.perf_counter() - t0
    st = ctx.stats()
    res["decode_gpu_ms_per_token"] = round(st["gpu_ms"] / max(1, st["n_calls"]), 4)
    res["prefill_tok_s"] = round(n_prompt / sorted(t_pre)[1], 1)
    res["decode_tok_s"] = round(n_decode / t_dec, 1)
    res["prefill_ms"] = round(sorted(t_pre)[1] * 1e3, 3)
    res["decode_ms_per_token"] = round(t_dec / n_decode * 1e3, 4)
    # kernel by kernel, eager launches (events inside a replayed graph cannot be read): one prompt pass, eight single tokens
    ctx.seq_rm(0, -1, -1)
    ctx.set_graphs(False)
    res["prefill_kernels"] = kernel_table(lib, lambda: ctx.feed(toks[:n_prompt], 0, 0))
    res["decode_kernels"] = kernel_table(lib, lambda: [ctx.feed(toks[n_prompt + i:n_prompt + i + 1], n_prompt + i, 0) for i in range(8)])
    ctx.free(); model.free()
    return res


def main_parallel(sizes, cache, n_prompt=512, n_decode=64):
    """Vikarax beside Fasovik at equal sizes; one JSON line per size"""
    lib = L.load()
    L.check(lib.pi_device_init(0), "pi_device_init")
    for size in sizes:
        width, n_layer, heads, dim, vdim, rank, n_exp, n_id, top, ff, vocab = SIZES[size]
        kv_heads, rot, chunk, r_heads, r_vdim, state, groups, g_count, g_keep, shared = VIKARAX[size]
        vik, fas = os.path.join(cache, "vikarax-" + size), os.path.join(cache, "fasovik-" + size)
        if not os.path.exists(os.path.join(vik, "model.safetensors")):
            write_vikarax(vik, size)
        if not os.path.exists(os.path.join(fas, "model.safetensors")):
            write_fasovik(fas, size)
        out = {"size": size, "config": {"width": width, "layers": n_layer, "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot_dims": rot, "chunk": chunk,
                                       "recurrence": {"heads": r_heads, "vdim": r_vdim, "state": state, "groups": groups, "conv": 4}, "experts": n_exp, "top": top, "ff": ff, "shared_ff": shared,
                                       "vocab": vocab, "n_prompt": n_prompt, "n_decode": n_decode, "fasovik": {"kv_rank": rank, "identity": n_id}},
               "vikarax_bf16": measure(lib, vik, n_prompt, n_decode, True),
               "fasovik_bf16": measure(lib, fas, n_prompt, n_decode, True), "data": "synthetic", "hbm_peak": HBM_PEAK}
        print(json.dumps(out))
        sys.stdout.flush()
    return 0


def main_postnorm(sizes, cache, n_prompt=512, n_decode=64):
    """Rafusun beside Vikarax (dense feed-forward of the same width) at equal sizes; one JSON line per size"""
    lib = L.load()
    L.check(lib.pi_device_init(0), "pi_device_init")
    for size in sizes:
        width, n_layer, heads, dim, vdim, _, _, _, _, ff, vocab = SIZES[size]
        kv_heads, rot, chunk, r_heads, r_vdim, state, groups, _, _, _ = VIKARAX[size]
        raf, vik = os.path.join(cache, "rafusun-" + size), os.path.join(cache, "vikarax-dense-" + size)
        if not os.path.exists(os.path.join(raf, "model.safetensors")):
            write_rafusun(raf, size)
        if not os.path.exists(os.path.join(vik, "model.safetensors")):
            write_vikarax(vik, size, dense_ff=4 * ff)
        out = {"size": size, "config": {"width": width, "layers": n_layer, "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot_dims": rot, "chunk": chunk, "conv": 4, "low_rank": 64,
                                       "time_mix": {"heads": r_heads, "dim": r_vdim}, "vikarax_recurrence": {"heads": r_heads, "vdim": r_vdim, "state": state, "groups": groups}, "ff": 4 * ff,
                                       "vocab": vocab, "n_prompt": n_prompt, "n_decode": n_decode},
               "rafusun_bf16": measure(lib, raf, n_prompt, n_decode, True),
               "vikarax_dense_bf16": measure(lib, vik, n_prompt, n_decode, True), "data": "synthetic", "hbm_peak": HBM_PEAK}
        print(json.dumps(out))
        sys.stdout.flush()
    return 0


def main_window(sizes, cache, n_prompt=512, n_decode=64):
    """Rarevik beside Vikarax (routed experts with a shared one) at equal sizes; one JSON line per size"""
    lib = L.load()
    L.check(lib.pi_device_init(0), "pi_device_init")
    for size in sizes:
        width, n_layer, heads, dim, vdim, _, n_exp, _, top, ff, vocab = SIZES[size]
        kv_heads, rot, chunk, r_heads, r_vdim, state, groups, _, _, shared = VIKARAX[size]
        pool, conv = RAREVIK[size]
        rar, vik = os.path.join(cache, "rarevik-" + size), os.path.join(cache, "vikarax-" + size)
        if not os.path.exists(os.path.join(rar, "model.safetensors")):
            write_rarevik(rar, size)
        if not os.path.exists(os.path.join(vik, "model.safetensors")):
            write_vikarax(vik, size)
        out = {"size": size, "config": {"width": width, "layers": n_layer, "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot_dims": rot, "window": chunk, "pool": pool, "conv": conv,
                                       "experts": n_exp, "top": top, "ff": ff, "shared_ff": shared, "vikarax_recurrence": {"heads": r_heads, "vdim": r_vdim, "state": state, "groups": groups},
                                       "vocab": vocab, "n_prompt": n_prompt, "n_decode": n_decode},
               "rarevik_bf16": measure(lib, rar, n_prompt, n_decode, True),
               "vikarax_bf16": measure(lib, vik, n_prompt, n_decode, True), "data": "synthetic", "hbm_peak": HBM_PEAK}
        print(json.dumps(out))
        sys.stdout.flush()
    return 0


def main(sizes, cache, n_prompt=512, n_decode=64):
    lib = L.load()
    L.check(lib.pi_device_init(0), "pi_device_init")
    from bench import ensure_model
    for size in sizes:
        width, n_layer, heads, dim, vdim, rank, n_exp, n_id, top, ff, vocab = SIZES[size]
        folder = os.path.join(cache, "fasovik-" + size)
        if not os.path.exists(os.path.join(folder, "model.safetensors")):
            write_fasovik(folder, size)
        n_ff = max(32, int(round(2 * top * ff / 3 / 32)) * 32)      # a gated Llama feed-forward with the parameters a token's chosen experts have
        spec = "cmp-llama-" + size
        synth.SPECS[spec] = ("llama", n_layer, width, heads, heads, n_ff, vocab, 4096)
        gguf = ensure_model(cache, spec, "q8_0", 0x5EED, 1.0, 0.25)
        out = {"size": size, "config": {"width": width, "layers": n_layer, "heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "experts": n_exp, "identity": n_id, "top": top,
                                       "ff": ff, "vocab": vocab, "n_prompt": n_prompt, "n_decode": n_decode, "llama_n_ff": n_ff},
               "fasovik_bf16": measure(lib, folder, n_prompt, n_decode, True),
               "llama_q8_0": measure(lib, gguf, n_prompt, n_decode, False), "data": "synthetic", "hbm_peak": HBM_PEAK}
        print(json.dumps(out))
        sys.stdout.flush()
    return 0


def run_phase(design, size, phase, cache, n_prompt=512, n_decode=64):
    """one phase of one design at one size and nothing else, for a profiler: `prefill` = four prompt passes, `decode` = one prompt pass and n_decode single tokens"""
    lib = L.load()
    L.check(lib.pi_device_init(0), "pi_device_init")
    folder = os.path.join(cache, "%s-%s" % (design, size))
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        {"vikarax": write_vikarax, "fasovik": write_fasovik, "rafusun": write_rafusun, "rarevik": write_rarevik}[design](folder, size)
    model = LL.Model(folder)
    ctx = LL.Context(model, n_ctx=n_prompt + n_decode + 64, n_batch=n_prompt)
    ctx.set_precision(False)
    rng = np.random.default_rng(7)
    toks = [int(t) for t in rng.integers(1, model.n_vocab, n_prompt + n_decode)]
    if phase == "prefill":
        for _ in range(4):
            ctx.feed(toks[:n_prompt], 0, 0)
            ctx.seq_rm(0, -1, -1)
    else:
        ctx.feed(toks[:n_prompt], 0, 0)
        for i in range(n_decode):
            ctx.feed(toks[n_prompt + i:n_prompt + i + 1], n_prompt + i, 0)
    ctx.free(); model.free()
    return 0


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description="one phase of one folder-described design at one size (for `rocprofv3 --kernel-trace --stats -- python3 -m pipeinfer_amd.tools.hybrid_bench ...`)")
    ap.add_argument("--design", choices=["vikarax", "fasovik", "rafusun", "rarevik"], required=True)
    ap.add_argument("--size", choices=sorted(SIZES), default="w2048")
    ap.add_argument("--phase", choices=["prefill", "decode"], required=True)
    ap.add_argument("--cache", default=os.environ.get("PIPEINFER_CACHE", "/tmp/pipeinfer_models"))
    a = ap.parse_args()
    sys.exit(run_phase(a.design, a.size, a.phase, a.cache))
