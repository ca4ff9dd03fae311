"""Plain, slow restatement of the Rarevik design in numpy (float64), one function per mechanism, token by token: the oracle the engine's kernels are held to.
It shares no code with the product path (file reading and bfloat16 rounding come from the other oracle of this folder, which is test infrastructure too).

A model is {"config": <the config.json dictionary>, "tensors": {name: float64 array}}.

Notation.  T(y; a, w, b) = tanh(a y) * w + b (a norm without statistics), R(y) = y / sqrt(mean(y^2) + eps).
Order:       layers [start, stop) of the list run `times` times with the same tensors (every run has a cache and state of its own), the others once.  In front of the first
             layer of every such run x <- W_in [x ; x0], x0 the embedding row.
A layer:     h = T(x);  m = h + (h_prev - h) * shift (h_prev: the previous token's h of this layer run, zeros at the start);  x <- x + mixer(m) + ff(h).
attention    q, k (G heads of D), v (G heads of V) = W m, each channel through a causal convolution over its last `conv` values (no bias, no activation);
             q, k <- R(.) * norm per head, then the first `dims` dimensions turned in pairs (i, i + dims/2) by pos * base^(-2i/dims);
             token i sees the tokens j with 0 <= i - j < size and, for every block b of P positions with bP + P - 1 <= i - size, ONE key and value: the means of the
             block's cached keys / values;  p = exp(s) / (exp(sink_h) + sum exp(s)) over both kinds, s = q.k * scale;  W_o.
attention_2  q, k, v = W m;  q, k turned in pairs (2i, 2i + 1), the frequencies stretched by wavelength (factor, low, high, original);  tokens 0 <= i - j < size;
             ordinary soft-max;  head h's output * sigmoid(W_g m)_h;  W_o.
Feed-forward dense: W_down gelu(W_up h) (erf form);  routed: z = W_r h + b, the `top` largest, weights = soft-max over those; expert e: g = min(W_gate h, L),
             u = clip(W_up h, -L, L), W_down (g sigmoid(1.702 g) (u + 1));  + sigmoid(W_sg h) * shared expert (same form, its own L).
Output:      embed @ T(x; final.norm).
"""
import math

import numpy as np

from tests.fasovik_oracle import bf16_round, read_model, write_model  # noqa: F401  (files and rounding: shared test infrastructure)

_erf = np.vectorize(math.erf, otypes=[np.float64])


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def gelu_erf(z):
    return 0.5 * z * (1.0 + _erf(z / math.sqrt(2.0)))


def tanh_norm(T, name, y):
    return np.tanh(float(T[name + ".alpha"]) * y) * T[name] + T[name + ".b"]


def unit_rms(y, eps):
    return y / np.sqrt((y * y).mean() + eps)


def shifted(h, prev, mu):
    return h + (prev - h) * mu


def short_conv(w, window, new):
    """w [channels][taps]; window: the last taps - 1 inputs, oldest first (list of arrays); returns the output and the new window"""
    taps = w.shape[1]
    seq = window + [new]
    out = sum(w[:, j] * seq[j] for j in range(taps))
    return out, seq[1:] if taps > 1 else []


def frequencies(rot):
    """one angle step per pair, stretched for long wavelengths where the description says so"""
    dims = rot["dims"]
    f = np.array([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)])
    sc = rot.get("scaling")
    if not sc:
        return f
    out = f.copy()
    for i, fi in enumerate(f):
        wl = 2.0 * math.pi / fi
        if wl < sc["original"] / sc["high"]:
            continue
        if wl > sc["original"] / sc["low"]:
            out[i] = fi / sc["factor"]
        else:
            s = (sc["original"] / wl - sc["low"]) / (sc["high"] - sc["low"])
            out[i] = (1.0 - s) * fi / sc["factor"] + s * fi
    return out


def rotate(vec, pos, rot, neighbours):
    """the first rot.dims entries of vec turned in pairs: (i, i + dims/2), or (2i, 2i + 1) with neighbours"""
    if not rot:
        return vec
    out = vec.copy()
    dims = rot["dims"]
    for i, fi in enumerate(frequencies(rot)):
        a = pos * fi
        ia, ib = (2 * i, 2 * i + 1) if neighbours else (i, i + dims // 2)
        u, v = vec[ia], vec[ib]
        out[ia], out[ib] = u * math.cos(a) - v * math.sin(a), v * math.cos(a) + u * math.sin(a)
    return out


def visible_entries(i, size, pool):
    """(tokens j, blocks b) that position i sees"""
    lo = 0 if not size else max(0, i - size + 1)
    toks = list(range(lo, i + 1))
    blocks = []
    if size and pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return toks, blocks


def softmax_with(scores, extra=None):
    """weights of the scores; extra: one more term of the denominator (a logit without a value)"""
    m = max(scores.max(), extra) if extra is not None else scores.max()
    e = np.exp(scores - m)
    den = e.sum() + (math.exp(extra - m) if extra is not None else 0.0)
    return e / den


def attention_step(T, p, c, eps, m, pos, st):
    """the mixer 'attention'"""
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q, k, v = T[p + "q"] @ m, T[p + "k"] @ m, T[p + "v"] @ m
    if c.get("conv"):
        for name in "qkv":
            win = st.setdefault("conv_" + name, [np.zeros(T[p + name].shape[0]) for _ in range(c["conv"] - 1)])
            y, st["conv_" + name] = short_conv(T[p + name + ".conv"], win, {"q": q, "k": k, "v": v}[name])
            if name == "q":
                q = y
            elif name == "k":
                k = y
            else:
                v = y
    q, k, v = q.reshape(H, D), k.reshape(G, D), v.reshape(G, V)
    q = np.stack([rotate(unit_rms(q[h], eps) * T[p + "q.norm"], pos, c.get("rot"), False) for h in range(H)])
    k = np.stack([rotate(unit_rms(k[g], eps) * T[p + "k.norm"], pos, c.get("rot"), False) for g in range(G)])
    st.setdefault("k", []).append(k)
    st.setdefault("v", []).append(v)
    mask = c.get("mask") or {}
    toks, blocks = visible_entries(pos, mask.get("size"), mask.get("pool"))
    P = mask.get("pool")
    out = np.zeros((H, V))
    for h in range(H):
        g = h // (H // G)
        keys = [st["k"][j][g] for j in toks] + [np.mean([st["k"][j][g] for j in range(b * P, b * P + P)], axis=0) for b in blocks]
        vals = [st["v"][j][g] for j in toks] + [np.mean([st["v"][j][g] for j in range(b * P, b * P + P)], axis=0) for b in blocks]
        s = np.array([q[h] @ kk for kk in keys]) * c["scale"]
        w = softmax_with(s, float(T[p + "sink"][h]))
        out[h] = sum(wi * vi for wi, vi in zip(w, vals))
    return T[p + "o"] @ out.reshape(-1)


def attention_2_step(T, p, c, eps, m, pos, st):
    """the mixer 'attention_2'"""
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q, k, v = (T[p + "q"] @ m).reshape(H, D), (T[p + "k"] @ m).reshape(G, D), (T[p + "v"] @ m).reshape(G, V)
    q = np.stack([rotate(q[h], pos, c.get("rot"), True) for h in range(H)])
    k = np.stack([rotate(k[g], pos, c.get("rot"), True) for g in range(G)])
    st.setdefault("k", []).append(k)
    st.setdefault("v", []).append(v)
    toks, _ = visible_entries(pos, (c.get("mask") or {}).get("size"), None)
    gate = sigmoid(T[p + "g"] @ m)
    out = np.zeros((H, V))
    for h in range(H):
        g = h // (H // G)
        s = np.array([q[h] @ st["k"][j][g] for j in toks]) * c["scale"]
        w = softmax_with(s)
        out[h] = gate[h] * sum(wi * st["v"][j][g] for wi, j in zip(w, toks))
    return T[p + "o"] @ out.reshape(-1)


def clipped_expert(T, p, limit, h):
    g, u = T[p + "gate"] @ h, T[p + "up"] @ h
    if limit is not None:
        g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
    return T[p + "down"] @ (g * sigmoid(1.702 * g) * (u + 1.0))


def route(T, p, top, h):
    z = T[p + "router"] @ h + T[p + "router.b"]
    order = sorted(range(len(z)), key=lambda e: (-z[e], e))[:top]
    return order, softmax_with(np.array([z[e] for e in order]))


def feed_forward(T, p, c, h):
    if c["kind"] == "dense":
        return T[p + "down"] @ gelu_erf(T[p + "up"] @ h)
    chosen, weights = route(T, p, c["router"]["top"], h)
    y = sum(w * clipped_expert(T, p + "e%d." % e, c["expert"].get("limit"), h) for e, w in zip(chosen, weights))
    if c.get("shared"):
        y = y + sigmoid(T[p + "shared.sg"] @ h)[0] * clipped_expert(T, p + "shared.", c["shared"].get("limit"), h)
    return y


def layer_runs(config):
    """[(layer index, first of a repeated run)] in the order the layers run"""
    n, loop = len(config["layers"]), config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def new_state():
    return {"pos": 0, "runs": {}}


def step(model, state, token, layers_out=None):
    """one token of one sequence through the model; returns the logits.  layers_out (a list) receives the stream after every layer run"""
    c, T = model["config"], model["tensors"]
    eps = c["norm"]["eps"]
    x0 = T["embed"][token].copy()
    x, pos = x0.copy(), state["pos"]
    for r, (i, entry) in enumerate(layer_runs(c)):
        L, p = c["layers"][i], "l%d." % i
        st = state["runs"].setdefault(r, {})
        if entry:
            x = T["loop.in"] @ np.concatenate([x, x0])
        h = tanh_norm(T, p + "norm1", x)
        m = shifted(h, st.get("prev", np.zeros_like(h)), T[p + "shift"])
        st["prev"] = h
        if L["type"] == "attention":
            y = attention_step(T, p + "mix.", L["mixer"], eps, m, pos, st)
        elif L["type"] == "attention_2":
            y = attention_2_step(T, p + "mix.", L["mixer"], eps, m, pos, st)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            y = y + feed_forward(T, p + "mlp.", L["mlp"], h)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.copy())
    state["pos"] = pos + 1
    return T["embed"] @ tanh_norm(T, "final.norm", x)


def run(model, tokens, state=None, layers=None):
    """logits [len(tokens)][vocab] of a sequence (continued from `state`); layers (a list) receives [layer runs][width] per token"""
    state = new_state() if state is None else state
    out = []
    for t in tokens:
        lo = [] if layers is not None else None
        out.append(step(model, state, int(t), lo))
        if layers is not None:
            layers.append(np.stack(lo))
    return np.stack(out)


def greedy(model, prompt, n):
    state = new_state()
    lg = run(model, prompt, state)[-1]
    out = []
    for _ in range(n):
        out.append(int(np.argmax(lg)))
        lg = step(model, state, out[-1])
    return out


# ---- random models for the tests ----------------------------------------------------------------------------------------------------
def window_layer(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, size=7, pool=3, rot_dims=4, rot_base=100.0, scale=0.5, mlp=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        mx["conv"] = conv
    if rot_dims:
        mx["rot"] = {"dims": rot_dims, "base": rot_base}
    if size:
        mx["mask"] = {"size": size}
        if pool:
            mx["mask"]["pool"] = pool
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def gated_layer(heads=4, kv_heads=2, dim=6, vdim=5, size=9, rot_dims=6, rot_base=50.0, scaling=(4.0, 1.0, 4.0, 64), scale=0.5, mlp=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot_dims:
        mx["rot"] = {"dims": rot_dims, "base": rot_base}
        if scaling:
            mx["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if size:
        mx["mask"] = {"size": size}
    return {"type": "attention_2", "mixer": mx, "mlp": mlp}


def dense_mlp(ff):
    return {"kind": "dense", "ff": ff}


def routed_mlp(experts=5, top=2, ff=6, limit=1.25, shared_ff=4, shared_limit=0.75):
    c = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared_ff:
        c["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return c


def random_model(rng, vocab, width, layers, loop=None, eps=1e-5):
    """weights rounded to bfloat16 (what the file holds), sized so that every mechanism matters in the logits"""
    def w(*shape, s=None):
        s = s if s is not None else 1.0 / np.sqrt(shape[-1])
        return bf16_round((rng.standard_normal(shape) * s).astype(np.float32)).astype(np.float64)

    def rb(a):
        return bf16_round(np.asarray(a, np.float32)).astype(np.float64)

    def near_one(n):
        return rb(1.0 + 0.3 * rng.standard_normal(n))

    def tanh_norm_tensors(name):
        T[name], T[name + ".b"], T[name + ".alpha"] = near_one(width), w(width, s=0.2), rb(0.6 + 0.5 * rng.random())

    def expert(p, ff):
        T[p + "gate"], T[p + "up"], T[p + "down"] = w(ff, width, s=2.0 / np.sqrt(width)), w(ff, width, s=2.0 / np.sqrt(width)), w(width, ff)

    T = {"embed": w(vocab, width, s=0.8)}
    tanh_norm_tensors("final.norm")
    if loop:
        T["loop.in"] = rb(np.concatenate([np.eye(width), np.zeros((width, width))], axis=1) * 0.7 + rng.standard_normal((width, 2 * width)) * 0.5 / np.sqrt(width))
    for i, L in enumerate(layers):
        p, mx, m = "l%d." % i, L["mixer"], "l%d.mix." % i
        tanh_norm_tensors(p + "norm1")
        T[p + "shift"] = rb(rng.uniform(0.0, 1.0, width))
        H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        T[m + "q"], T[m + "k"], T[m + "v"], T[m + "o"] = w(H * D, width), w(G * D, width), w(G * V, width), w(width, H * V)
        if L["type"] == "attention":
            if mx.get("conv"):
                for n, rows in (("q", H * D), ("k", G * D), ("v", G * V)):
                    T[m + n + ".conv"] = w(rows, mx["conv"], s=0.7)
            T[m + "q.norm"], T[m + "k.norm"] = near_one(D), near_one(D)
            T[m + "sink"] = w(H, s=1.0)
        else:
            T[m + "g"] = w(H, width, s=2.0 / np.sqrt(width))
        c = L.get("mlp")
        if c and c["kind"] == "dense":
            T[p + "mlp.up"], T[p + "mlp.down"] = w(c["ff"], width), w(width, c["ff"])
        elif c:
            for e in range(c["router"]["experts"]):
                expert(p + "mlp.e%d." % e, c["expert"]["ff"])
            T[p + "mlp.router"], T[p + "mlp.router.b"] = w(c["router"]["experts"], width, s=2.0 / np.sqrt(width)), w(c["router"]["experts"], s=0.5)
            if c.get("shared"):
                expert(p + "mlp.shared.", c["shared"]["ff"])
                T[p + "mlp.shared.sg"] = w(1, width)
    config = {"architecture": "Rarevik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": [dict(L) for L in layers]}
    if loop:
        config["loop"] = dict(zip(("start", "stop", "times"), loop))
    return {"config": config, "tensors": T}
