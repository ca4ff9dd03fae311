"""Plain, slow restatement of the Rafusun design in numpy (float64), one function per mechanism, token by token: the oracle the engine's kernels are held to.
It shares no code with the product path (file reading and bfloat16 rounding come from the other oracle of this folder, which is test infrastructure too).

A model is {"config": <the config.json dictionary>, "tensors": {name: float64 array}}.

Notation.  R(y) = y / sqrt(mean(y^2) + eps), U(y) = y / sqrt(sum(y^2) + 1e-6).
Embedding:   x = embed[t] * scale + bigram[(t_prev * mul_prev + t * mul_cur) mod buckets]; the first token of a sequence takes the table's last row.
A layer:     x <- R(alpha x + ls1 * mixer(x)) * norm1;   with a feed-forward also   x <- R(alpha x + ls2 * ff(x)) * norm2.   The sublayers read x itself.
channel_delta  q, k (G heads of D), v (H heads of V) = silu(conv(W h)): a causal convolution per channel over the last `conv` inputs; q = U(q) / sqrt(D), k = U(k) per head;
             beta = sigmoid(W_b h);  g = exp(-exp(A_log_h) softplus(W_a2 W_a1 h + dt_bias)) per head and key channel;
             S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;   out = W_o [R(o_h) * norm * sigmoid(W_g2 W_g1 h)_h].
parallel     0.5 (R(left(h)) * left.out + R(right(h)) * right.out).
  left       soft-max attention, H query heads over G key/value heads; q, k: the first `dims` dimensions turned in pairs (2i, 2i+1) by pos * base^(-2i/dims), then R(.) per head;
             s = cap tanh(q.k scale / cap) for the keys j <= i of the same block of `size` positions; p_j = exp(s_j) / (1 + sum exp(s)); W_o.
  right      m_s = h + (h_prev - h) mu_s for s in r, k, v, g, w;  r, k, v = W m;  gate = silu(W_g m_g);  w = exp(-exp(W_w2 tanh(W_w1 m_w) + w0));
             o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T;   out = W_o [R(o_h) * norm * gate].
Feed-forward: W_down (gelu_tanh(W_gate h) * W_up h).
Output:      W_head (R(x) * final.norm).
"""
import numpy as np

from tests.fasovik_oracle import bf16_round, read_model, write_model  # noqa: F401  (files and rounding: shared test infrastructure)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(y, eps):
    return y / np.sqrt((y * y).mean() + eps)


def unit_length(y):
    return y / np.sqrt((y * y).sum() + 1e-6)


def rotate_pairs(vec, pos, dims, base):
    """the first `dims` entries of vec, neighbours (2i, 2i + 1) as pairs, turned by pos * base^(-2i/dims)"""
    out = vec.copy()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        u, v = vec[2 * i], vec[2 * i + 1]
        out[2 * i], out[2 * i + 1] = u * np.cos(a) - v * np.sin(a), v * np.cos(a) + u * np.sin(a)
    return out


def embed(model, token, prev):
    c, T = model["config"], model["tensors"]
    b = c["embedding"]["bigram"]
    row = b["buckets"] if prev is None else (prev * b["mul_prev"] + token * b["mul_cur"]) % b["buckets"]
    return T["embed"][token] * c["embedding"]["scale"] + T["bigram"][row]


def short_conv(w, window, new):
    """window: the last taps - 1 inputs [taps - 1][channels] (oldest first); returns the convolution at the new input and the next window"""
    full = np.concatenate([window, new[None, :]], axis=0)
    out = (full * w.T).sum(axis=0)
    return out, full[1:]


def channel_delta_step(T, p, c, eps, h, st):
    """one token; st: {"S": [H][D][V], "conv": {"q" | "k" | "v": [taps - 1][channels]}}"""
    H, G, D, V, taps = c["heads"], c["kv_heads"], c["dim"], c["vdim"], c["conv"]
    if not st:
        st["S"] = np.zeros((H, D, V))
        st["conv"] = {n: np.zeros((taps - 1, (H if n == "v" else G) * (V if n == "v" else D))) for n in "qkv"}
    z = {}
    for n in "qkv":
        z[n], st["conv"][n] = short_conv(T[p + n + ".conv"], st["conv"][n], T[p + n] @ h)
        z[n] = silu(z[n])
    q, k, v = z["q"].reshape(G, D), z["k"].reshape(G, D), z["v"].reshape(H, V)
    beta = sigmoid(T[p + "b"] @ h)
    g = np.exp(-np.exp(T[p + "A_log"])[:, None] * softplus(T[p + "a2"] @ (T[p + "a1"] @ h) + T[p + "dt_bias"]).reshape(H, D))
    gate = sigmoid(T[p + "g2"] @ (T[p + "g1"] @ h)).reshape(H, V)
    out = np.zeros((H, V))
    for i in range(H):
        j = i // (H // G)
        qi, ki = unit_length(q[j]) * D ** -0.5, unit_length(k[j])
        S = st["S"][i] * g[i][:, None]
        u = beta[i] * (v[i] - S.T @ ki)
        S = S + np.outer(ki, u)
        st["S"][i] = S
        out[i] = unit_rms(S.T @ qi, eps) * T[p + "norm"] * gate[i]
    return T[p + "o"] @ out.reshape(-1)


def softmax_attention_step(T, p, c, eps, h, pos, st):
    """one token of the attention branch; st["kv"]: [(position, keys [G][D], values [G][V]), ...] of the sequence so far; this token's are appended"""
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    rot = c.get("rot") or {"dims": 0, "base": 1.0}
    q = (T[p + "q"] @ h).reshape(H, D)
    k = (T[p + "k"] @ h).reshape(G, D)
    v = (T[p + "v"] @ h).reshape(G, V)
    q = np.stack([unit_rms(rotate_pairs(q[i], pos, rot["dims"], rot["base"]), eps) for i in range(H)])
    k = np.stack([unit_rms(rotate_pairs(k[i], pos, rot["dims"], rot["base"]), eps) for i in range(G)])
    st.setdefault("kv", []).append((pos, k, v))
    size = (c.get("mask") or {}).get("size")
    cap = c.get("softcap")
    out = np.zeros((H, V))
    for i in range(H):
        g = i // (H // G)
        seen = [(kj[g], vj[g]) for pj, kj, vj in st["kv"] if pj <= pos and not (size and pj // size != pos // size)]
        s = np.array([q[i] @ kj for kj, _ in seen]) * c["scale"]
        if cap:
            s = cap * np.tanh(s / cap)
        e = np.exp(s)
        w = e / (1.0 + e.sum())
        out[i] = sum(wj * vj for wj, (_, vj) in zip(w, seen))
    return T[p + "o"] @ out.reshape(-1)


def time_mix_step(T, p, c, eps, h, st):
    """one token of the time-mixing branch; st: {"S": [H][D][D], "prev": the previous token's h}"""
    H, D = c["heads"], c["dim"]
    if "S" not in st:
        st["S"] = np.zeros((H, D, D))
        st["prev"] = np.zeros_like(h)
    m = {n: h + (st["prev"] - h) * T[p + "mu." + n] for n in "rkvgw"}
    st["prev"] = h.copy()
    r, k, v = ((T[p + n] @ m[n]).reshape(H, D) for n in "rkv")
    gate = silu(T[p + "g"] @ m["g"])
    w = np.exp(-np.exp(T[p + "w2"] @ np.tanh(T[p + "w1"] @ m["w"]) + T[p + "w0"])).reshape(H, D)
    out = np.zeros((H, D))
    for i in range(H):
        kv = np.outer(k[i], v[i])
        out[i] = unit_rms((st["S"][i] + T[p + "u"][i][:, None] * kv).T @ r[i], eps)
        st["S"][i] = w[i][:, None] * st["S"][i] + kv
    return T[p + "o"] @ (out.reshape(-1) * T[p + "norm"] * gate)


def parallel_step(T, p, c, eps, h, pos, st):
    a = softmax_attention_step(T, p + "left.", c["left"], eps, h, pos, st.setdefault("left", {}))
    b = time_mix_step(T, p + "right.", c["right"], eps, h, st.setdefault("right", {}))
    return 0.5 * (unit_rms(a, eps) * T[p + "left.out"] + unit_rms(b, eps) * T[p + "right.out"])


def feed_forward(T, p, h):
    return T[p + "down"] @ (gelu_tanh(T[p + "gate"] @ h) * (T[p + "up"] @ h))


def new_state():
    return {"pos": 0, "prev": None, "layers": {}}


def step(model, state, token, layers_out=None):
    """one token of one sequence through the model; returns the logits.  layers_out (a list) receives the stream after every layer"""
    c, T = model["config"], model["tensors"]
    eps, alpha = c["norm"]["eps"], c["postln_alpha"]
    x = embed(model, token, state["prev"])
    pos = state["pos"]
    for i, L in enumerate(c["layers"]):
        p = "l%d." % i
        st = state["layers"].setdefault(i, {})
        if L["type"] == "channel_delta":
            y = channel_delta_step(T, p + "mix.", L["mixer"], eps, x, st)
        elif L["type"] == "parallel":
            y = parallel_step(T, p + "mix.", L["mixer"], eps, x, pos, st)
        else:
            raise ValueError(L["type"])
        x = unit_rms(alpha * x + T[p + "ls1"] * y, eps) * T[p + "norm1"]
        if L.get("mlp"):
            x = unit_rms(alpha * x + T[p + "ls2"] * feed_forward(T, p + "mlp.", x), eps) * T[p + "norm2"]
        if layers_out is not None:
            layers_out.append(x.copy())
    state["pos"], state["prev"] = pos + 1, token
    return T["head"] @ (unit_rms(x, eps) * T["final.norm"])


def run(model, tokens, state=None, layers=None):
    """logits [len(tokens)][vocab] of a sequence (continued from `state`); layers (a list) receives [layers][width] per token"""
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
def delta_layer(heads=2, kv_heads=1, dim=6, vdim=5, conv=3, decay_rank=3, gate_rank=2, mlp=None):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp, "_ranks": (decay_rank, gate_rank)}


def parallel_layer(heads=4, kv_heads=2, dim=6, vdim=5, chunk=7, rot_dims=4, rot_base=100.0, scale=0.5, softcap=8.0, r_heads=3, r_dim=4, decay_rank=2, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        left["softcap"] = softcap
    if rot_dims:
        left["rot"] = {"dims": rot_dims, "base": rot_base}
    if chunk:
        left["mask"] = {"size": chunk}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": r_heads, "dim": r_dim}}, "mlp": mlp, "_ranks": (decay_rank,)}


def dense_mlp(ff):
    return {"kind": "dense", "ff": ff}


def random_model(rng, vocab, width, layers, eps=1e-5, alpha=1.7, embed_scale=3.0, buckets=53, mul_prev=31, mul_cur=5):
    """weights rounded to bfloat16 (what the file holds), sized so that every mechanism matters in the logits"""
    def w(*shape, s=None):
        s = s if s is not None else 1.0 / np.sqrt(shape[-1])
        return bf16_round((rng.standard_normal(shape) * s).astype(np.float32)).astype(np.float64)

    def rb(a):
        return bf16_round(np.asarray(a, np.float32)).astype(np.float64)

    def near_one(n):
        return bf16_round((1.0 + 0.3 * rng.standard_normal(n)).astype(np.float32)).astype(np.float64)

    T = {"embed": w(vocab, width, s=0.4), "bigram": w(buckets + 1, width, s=0.8), "head": w(vocab, width), "final.norm": near_one(width)}
    cfg_layers = []
    for i, L in enumerate(layers):
        p = "l%d." % i
        L = dict(L)
        ranks = L.pop("_ranks")
        cfg_layers.append(L)
        T[p + "norm1"], T[p + "ls1"] = near_one(width), rb(w(width, s=0.5) + 1.0)
        mx, m = L["mixer"], p + "mix."
        if L["type"] == "channel_delta":
            H, G, D, V, taps = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["conv"]
            for n, rows in (("q", G * D), ("k", G * D), ("v", H * V)):
                T[m + n] = w(rows, width)
                T[m + n + ".conv"] = w(rows, taps, s=0.7)
            T[m + "b"] = w(H, width)
            T[m + "A_log"] = w(H, s=0.5)
            T[m + "dt_bias"] = rb(w(H * D, s=1.0) - 1.0)
            T[m + "a1"], T[m + "a2"] = w(ranks[0], width), w(H * D, ranks[0])
            T[m + "g1"], T[m + "g2"] = w(ranks[1], width), w(H * V, ranks[1])
            T[m + "norm"] = near_one(V)
            T[m + "o"] = w(width, H * V)
        else:
            A, R = mx["left"], mx["right"]
            T[m + "left.q"] = w(A["heads"] * A["dim"], width)
            T[m + "left.k"] = w(A["kv_heads"] * A["dim"], width)
            T[m + "left.v"] = w(A["kv_heads"] * A["vdim"], width)
            T[m + "left.o"] = w(width, A["heads"] * A["vdim"])
            T[m + "left.out"], T[m + "right.out"] = near_one(width), near_one(width)
            inner = R["heads"] * R["dim"]
            for n in "rkvgw":
                T[m + "right.mu." + n] = bf16_round(rng.uniform(0.0, 1.0, width).astype(np.float32)).astype(np.float64)
            for n in "rkvg":
                T[m + "right." + n] = w(inner, width)
            T[m + "right.w1"], T[m + "right.w2"] = w(ranks[0], width), w(inner, ranks[0])
            T[m + "right.w0"] = rb(w(inner, s=1.0) - 1.5)
            T[m + "right.u"] = w(R["heads"], R["dim"], s=0.7)
            T[m + "right.norm"] = near_one(inner)
            T[m + "right.o"] = w(width, inner)
        if L.get("mlp"):
            ff = L["mlp"]["ff"]
            T[p + "norm2"], T[p + "ls2"] = near_one(width), rb(w(width, s=0.5) + 1.0)
            T[p + "mlp.gate"], T[p + "mlp.up"], T[p + "mlp.down"] = w(ff, width), w(ff, width), w(width, ff)
    config = {"architecture": "Rafusun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
              "embedding": {"scale": embed_scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}, "layers": cfg_layers}
    return {"config": config, "tensors": T}
