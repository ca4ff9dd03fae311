"""The Rarevik design (one tanh norm per layer that a token-shifted mixer and the feed-forward both read, a run of layers repeated with the same tensors, sliding-window attention with a
short convolution, pooled far blocks and a learned sink, or with stretched rotation steps and a per-head gate; a dense or a routed feed-forward of clipped gated experts with a gated
shared expert) on the engine, held to the plain numpy restatement in tests/rarevik_oracle.py: every mechanism alone through its operator, then whole models through llama_decode —
prompts against token-by-token decoding, portions down to two tokens, batches of unequal requests, cells and state slots freed and used again, keys at the borders of windows and
pooled blocks, long decoding, greedy generation, the trace runner.  Models are small, random and made here; sizes are chosen so that nothing that could be mixed up is equal."""
import ctypes as C
import json
import math
import os

import numpy as np
import pytest

from pipeinfer_amd import lib as L, llama as LL
from tests import rarevik_oracle as O

BF16 = 30
F = 1 << 30                                    # "this sequence starts from nothing" on the first token of a run (slot words)
NONE, SILU, SIGMOID, GELU_ERF = 0, 1, 2, 6
SOFTMAX = 1
CHUNK, WINDOW = 0, 1
NORM_LAST, NORM_FIRST, NORM_NONE = 0, 1, 2
HALVES, NEIGHBOURS = 0, 1
GLU_OFF, GLU_SILU, GLU_CLIPPED = 0, 1, 2


def rel_rms(got, want):
    d = np.asarray(got, np.float64) - np.asarray(want, np.float64)
    return float(np.sqrt((d * d).mean()) / (np.sqrt((np.asarray(want, np.float64) ** 2).mean()) + 1e-30))


def logit_err(got, want):
    d = np.asarray(got, np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / (want - want.mean(-1, keepdims=True)).std()


TOL = {True: 3e-4, False: 4e-2}          # exact (fp32) / serving precision (bfloat16 matrix inputs)


def within(err, exact, tol=None):
    """fp32: every position within the tolerance.  Serving precision is held to the float64 restatement too, whose distance is the rounding of bfloat16 matrix inputs — and now and then
    a router's near tie that falls the other way: nine positions in ten within the tolerance; the fp32 runs of the same tests are the sharp ones"""
    tol = tol if tol is not None else TOL[exact]
    if exact:
        return err.max() < tol
    return np.quantile(err, 0.9) < tol


VOCAB = 83
# layer mixes: the default one, the values another model may make equal or one, wide heads, one kind of layer only, and the ways a run can repeat
VARIANTS = {
    "mixed": (None, (1, 3, 2)),
    "edges": ([O.window_layer(heads=1, kv_heads=1, dim=2, vdim=1, conv=1, size=1, pool=1, rot_dims=2, mlp=O.dense_mlp(1)),
               O.gated_layer(heads=1, kv_heads=1, dim=2, vdim=3, size=None, rot_dims=2, scaling=None, mlp=O.routed_mlp(experts=1, top=1, ff=1, limit=None, shared_ff=1, shared_limit=None)),
               O.window_layer(heads=2, kv_heads=2, dim=4, vdim=4, conv=None, size=None, pool=None, rot_dims=None, mlp=None),
               O.gated_layer(heads=3, kv_heads=3, dim=4, vdim=4, size=1, rot_dims=None, mlp=O.routed_mlp(experts=3, top=3, ff=5, shared_ff=None)),
               O.window_layer(heads=2, kv_heads=1, dim=6, vdim=2, conv=2, size=3, pool=None, rot_dims=6, mlp=O.routed_mlp(experts=4, top=1, ff=3))], (0, 5, 1)),
    "wide_heads": ([O.window_layer(heads=6, kv_heads=2, dim=72, vdim=66, conv=4, size=19, pool=4, rot_dims=40, scale=0.15, mlp=O.dense_mlp(50)),
                    O.gated_layer(heads=4, kv_heads=1, dim=130, vdim=10, size=33, rot_dims=130 - 2, scale=0.1, scaling=(8.0, 1.0, 2.0, 40), mlp=O.routed_mlp(experts=6, top=2, ff=16, shared_ff=24))], (0, 1, 2)),
    "only_window": ([O.window_layer(mlp=None), O.window_layer(heads=3, kv_heads=1, dim=8, vdim=4, conv=5, size=4, pool=6, rot_dims=6, mlp=O.dense_mlp(12))], None),
    "only_gated": ([O.gated_layer(mlp=O.routed_mlp()), O.gated_layer(heads=2, kv_heads=1, dim=10, vdim=3, size=5, rot_dims=4, scaling=(2.0, 0.5, 3.0, 16), mlp=None)], (1, 2, 3)),
    "repeat_all": ([O.gated_layer(mlp=O.dense_mlp(9)), O.window_layer(size=5, pool=2, mlp=None)], (0, 2, 3)),
}


def default_layers():
    return [O.window_layer(mlp=O.dense_mlp(24)),
            O.gated_layer(mlp=O.routed_mlp()),
            O.window_layer(heads=2, kv_heads=2, dim=10, vdim=4, conv=4, size=16, pool=5, rot_dims=2, mlp=O.routed_mlp(experts=7, top=3, ff=5, limit=0.9, shared_ff=None)),
            O.gated_layer(heads=6, kv_heads=2, dim=4, vdim=7, size=12, rot_dims=4, scaling=(3.0, 1.0, 2.0, 8), mlp=None)]


def small_model(seed=0, width=40, vocab=VOCAB, layers=None, loop=(1, 3, 2), **kw):
    rng = np.random.default_rng(seed)
    return O.random_model(rng, vocab, width, layers or default_layers(), loop=loop, **kw)


def variant_model(name, seed=11):
    layers, loop = VARIANTS[name]
    return small_model(seed=seed, layers=layers, loop=loop, width=64 if name == "wide_heads" else 40)


def write(folder, m):
    O.write_model(folder, m["config"], {k: v.astype(np.float32) for k, v in m["tensors"].items()})


class Engine:
    def __init__(self, tmp_path, model, n_ctx=256, n_batch=64, exact=True, slots=4, name="m"):
        folder = os.path.join(str(tmp_path), name)
        write(folder, model)
        self.model = LL.Model(folder)
        self.ctx = LL.Context(self.model, n_ctx=n_ctx, n_batch=n_batch)
        self.ctx.set_state_slots(slots)
        self.ctx.set_precision(exact)

    def close(self):
        self.ctx.free()
        self.model.free()


# ---- without a GPU ---------------------------------------------------------------------------------------------------------------
def test_model_folder_is_read_and_described(tmp_path):
    m = small_model()
    folder = str(tmp_path / "m")
    write(folder, m)
    mod = LL.Model(folder)
    assert mod.n_vocab == VOCAB
    buf = C.create_string_buffer(64)
    mod.lib.llama_model_desc.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
    mod.lib.llama_model_desc(mod.h, buf, 64)
    assert buf.value.lower().startswith(b"rarevik")
    mod.free()
    for name in VARIANTS:                                            # descriptions without a window, pooled blocks, a convolution, a rotation, limits, a shared expert, a feed-forward or a repeated run are read as well
        if VARIANTS[name][0]:
            write(str(tmp_path / name), variant_model(name, seed=1))
            LL.Model(str(tmp_path / name)).free()


@pytest.mark.parametrize("breakage", ["type", "kv_heads", "rot", "kind", "top", "loop", "pool", "scaling"])
def test_a_wrong_description_is_refused(tmp_path, breakage):
    m = small_model()
    cfg = json.loads(json.dumps(m["config"]))
    tensors = dict(m["tensors"])
    if breakage == "type":
        cfg["layers"][0]["type"] = "attention_3"
    elif breakage == "kv_heads":
        cfg["layers"][1]["mixer"]["kv_heads"] = 3
    elif breakage == "rot":
        cfg["layers"][0]["mixer"]["rot"]["dims"] = 5
    elif breakage == "kind":
        cfg["layers"][0]["mlp"]["kind"] = "sparse"
    elif breakage == "top":
        cfg["layers"][1]["mlp"]["router"]["top"] = 6
    elif breakage == "loop":
        cfg["loop"]["stop"] = 5
    elif breakage == "pool":
        cfg["layers"][0]["mixer"]["mask"]["pool"] = 0
    elif breakage == "scaling":
        del cfg["layers"][1]["mixer"]["rot"]["scaling"]["low"]
    folder = str(tmp_path / "bad")
    O.write_model(folder, cfg, {k: v.astype(np.float32) for k, v in tensors.items()})
    with pytest.raises(L.PipeInferError):
        LL.Model(folder)


@pytest.mark.gpu
@pytest.mark.parametrize("breakage", ["missing", "shape", "scalar"])
def test_a_wrong_tensor_is_refused_when_the_weights_load(tmp_path, breakage):
    m = small_model()
    tensors = dict(m["tensors"])
    if breakage == "missing":
        del tensors["l0.mix.sink"]
    elif breakage == "shape":
        tensors["l1.shift"] = tensors["l1.shift"][:-1]
    else:
        tensors["l2.norm1.alpha"] = np.ones(2)
    folder = str(tmp_path / "bad")
    O.write_model(folder, m["config"], {k: v.astype(np.float32) for k, v in tensors.items()})
    mod = LL.Model(folder)
    ctx = LL.Context(mod, n_ctx=32, n_batch=8)
    with pytest.raises(L.PipeInferError):
        ctx.decode([1], [0], [[0]])
    ctx.free()
    mod.free()


def test_oracle_mechanisms_behave_as_stated():
    """the restatement itself: what a position sees (the window's first position, a block the moment it lies wholly behind the window), rotations that keep lengths and depend on the
    distance only, stretched angle steps, a sink that takes its share, router weights over the chosen only, the order of repeated runs"""
    assert O.visible_entries(9, 4, 3) == ([6, 7, 8, 9], [0, 1])       # 9 - 4 = 5: block 1 (positions 3, 4, 5) ends there and is seen, block 2 would end at 8
    assert O.visible_entries(11, 4, 3)[1] == [0, 1] and O.visible_entries(8, 4, 3) == ([5, 6, 7, 8], [0]) and O.visible_entries(5, 4, 3)[1] == []      # (at 8 positions 3 and 4 are seen by nobody)
    assert O.visible_entries(6, 4, 3) == ([3, 4, 5, 6], [0]) and O.visible_entries(5, 4, 3) == ([2, 3, 4, 5], [])       # position 6: block 0 (ends at 2 = 6 - 4) is just seen; at 5 not yet, and position 1 is seen by nobody
    assert O.visible_entries(3, None, None) == ([0, 1, 2, 3], []) and O.visible_entries(7, 1, 1) == ([7], list(range(7)))
    rng = np.random.default_rng(3)
    for neighbours in (False, True):
        rot = {"dims": 6, "base": 100.0}
        v = rng.standard_normal(8)
        r = O.rotate(v, 11, rot, neighbours)
        ia, ib = (0, 1) if neighbours else (0, 3)
        assert np.isclose(np.linalg.norm(r), np.linalg.norm(v)) and np.array_equal(r[6:], v[6:]) and np.isclose(np.hypot(r[ia], r[ib]), np.hypot(v[ia], v[ib]))
        a, b = rng.standard_normal(6), rng.standard_normal(6)
        assert np.isclose(O.rotate(a, 9, rot, neighbours) @ O.rotate(b, 5, rot, neighbours), O.rotate(a, 104, rot, neighbours) @ O.rotate(b, 100, rot, neighbours))
    f = O.frequencies({"dims": 8, "base": 10000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}})
    plain = O.frequencies({"dims": 8, "base": 10000.0})
    wl = 2 * math.pi / plain                                          # 6.3, 63, 628, 6283: below 64 / 4 kept, above 64 / 1 divided, 63 between the two
    assert f[0] == plain[0] and np.isclose(f[2], plain[2] / 4) and np.isclose(f[3], plain[3] / 4) and plain[1] / 4 < f[1] < plain[1] and wl[1] < 64
    w = O.softmax_with(np.array([0.0, 0.0]), 0.0)
    assert np.allclose(w, [1 / 3, 1 / 3]) and np.allclose(O.softmax_with(np.array([1.0, 1.0])), [0.5, 0.5]) and O.softmax_with(np.array([0.0]), 50.0)[0] < 1e-20
    T = {"r.router": np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0], [-1.0, 0.0]]), "r.router.b": np.array([0.0, 0.0, -0.5, 5.0])}
    chosen, weights = O.route(T, "r.", 2, np.array([2.0, 1.0]))      # logits 2, 1, 2.5, 3: the last two win
    assert chosen == [3, 2] and np.allclose(weights, np.exp([3.0, 2.5]) / np.exp([3.0, 2.5]).sum())
    assert O.layer_runs({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 2}}) == [(0, False), (1, True), (2, False), (1, True), (2, False), (3, False), (4, False)]
    assert O.layer_runs({"layers": [0] * 2}) == [(0, False), (1, False)]
    g = np.array([3.0, -3.0, 0.5])
    T2 = {"e.gate": np.eye(3), "e.up": np.eye(3) * -1.0, "e.down": np.eye(3)}
    y = O.clipped_expert(T2, "e.", 1.0, g)                            # the gate is bounded from above only, the other half on both sides
    assert np.allclose(y, [1.0 * O.sigmoid(1.702) * (-1.0 + 1.0), -3.0 * O.sigmoid(-3.0 * 1.702) * (1.0 + 1.0), 0.5 * O.sigmoid(0.851) * 0.5])


# ---- operators alone ---------------------------------------------------------------------------------------------------------------
def gpu():
    from tests import gpu_util as U
    return U, U.init()


def upload_bf16(lib, w):
    u = (np.ascontiguousarray(w, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    h = lib.pi_weight_upload(BF16, w.shape[1], w.shape[0], u.ctypes.data_as(C.c_void_p), None)
    assert h, lib.pi_last_error()
    return h


def pack_mask(vis, n_kv):
    words = (n_kv + 31) // 32
    m = np.zeros((vis.shape[0], words), np.uint32)
    for t, j in zip(*np.nonzero(vis)):
        m[t, j >> 5] |= np.uint32(1 << (j & 31))
    return m


@pytest.mark.gpu
def test_dense_epilogue_erf_gelu():
    U, lib = gpu()
    rng = np.random.default_rng(2)
    W, x = O.bf16_round(rng.standard_normal((11, 24)).astype(np.float32)), (rng.standard_normal((5, 24)) * 2).astype(np.float32)
    w, xd, od = upload_bf16(lib, W), U.Dev(x), U.Dev(nbytes=4 * 5 * 11)
    L.check(lib.pi_op_dense(w, xd.ptr, 24, 5, od.ptr, 11, GELU_ERF, 6, NONE, 1, None))
    z = x.astype(np.float64) @ W.T.astype(np.float64)
    assert rel_rms(od.get(np.float32, (5, 11)), np.concatenate([O.gelu_erf(z[:, :6]), z[:, 6:]], axis=1)) < 2e-6
    lib.pi_weight_free(w)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [5, 300, 1030])
def test_layer_end_sum_norm_and_shift(n):
    """x + a + b + c with any of the three absent, in place; the tanh norm; its token shift over three sequences in passes of 1..40 tokens (both entries), a slot handed on over garbage"""
    U, lib = gpu()
    rng = np.random.default_rng(n)
    alpha = np.array([0.7], np.float32)
    w, bias, mu = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32), rng.uniform(0, 1, n).astype(np.float32)
    wd, bd, md, ad = U.Dev(w), U.Dev(bias), U.Dev(mu), U.Dev(alpha)
    slots = 3
    state = U.Dev((rng.standard_normal((slots, n)) * 50).astype(np.float32))
    prev = {}
    plan = [[(0, 5, True), (2, 1, True)], [(2, 40, False), (0, 2, False)], [(1, 3, True)], [(0, 1, False), (1, 1, False), (2, 1, False)], [(1, 36, True), (0, 33, False)]]
    for k, step in enumerate(plan):
        T = sum(c for _, c, _ in step)
        x, a, b, c = ((rng.standard_normal((T, n + 2)) * 2).astype(np.float32) for _ in range(4))
        use = [(k >> i) & 1 or k == 4 for i in range(3)]
        s64 = x[:, :n].astype(np.float64) + sum(v[:, :n].astype(np.float64) for v, u in zip((a, b, c), use) if u)
        h = np.tanh(0.7 * s64) * w + bias
        rec, want, at = [], np.zeros((T, n)), 0
        for slot, count, fresh in step:
            if fresh:
                prev[slot] = np.zeros(n)
            for i in range(count):
                rec.append(slot | (F if fresh and i == 0 else 0))
                want[at] = h[at] + (prev[slot] - h[at]) * mu
                prev[slot] = h[at]
                at += 1
        xd, da, db, dc, rd = U.Dev(x), U.Dev(a), U.Dev(b), U.Dev(c), U.Dev(np.array(rec, np.int32))
        hd, od = U.Dev(nbytes=4 * T * n), U.Dev(nbytes=4 * T * (n + 1))
        ptr = [d.ptr if u else None for d, u in zip((da, db, dc), use)]
        L.check(lib.pi_op_sum_tanh_norm_shift(xd.ptr, n + 2, ptr[0], n + 2, ptr[1], n + 2, ptr[2], n + 2, n, T, xd.ptr, n + 2, ad.ptr, wd.ptr, bd.ptr, hd.ptr, n, md.ptr, state.ptr, rd.ptr, od.ptr, n + 1, None))
        assert rel_rms(xd.get(np.float32, (T, n + 2))[:, :n], s64) < 1e-6 and np.array_equal(xd.get(np.float32, (T, n + 2))[:, n:], x[:, n:])
        assert rel_rms(hd.get(np.float32, (T, n)), h) < 3e-6 and rel_rms(od.get(np.float32, (T, n + 1))[:, :n], want) < 3e-6
        # the plain entry: no shift, the sum alone (no norm), the norm alone (no stream output)
        x2, h2 = U.Dev(nbytes=4 * T * n), U.Dev(nbytes=4 * T * n)
        L.check(lib.pi_op_sum_tanh_norm(xd.ptr, n + 2, None, 0, None, 0, None, 0, n, T, x2.ptr, n, None, None, None, None, 0, None))
        assert np.array_equal(x2.get(np.float32, (T, n)), xd.get(np.float32, (T, n + 2))[:, :n])
        L.check(lib.pi_op_sum_tanh_norm(xd.ptr, n + 2, None, 0, None, 0, None, 0, n, T, None, 0, ad.ptr, wd.ptr, None, h2.ptr, n, None))
        assert rel_rms(h2.get(np.float32, (T, n)), np.tanh(0.7 * s64) * w) < 3e-6
    st = state.get(np.float32, (slots, n))
    for slot in range(3):
        assert rel_rms(st[slot], prev[slot]) < 3e-6
    src = (rng.standard_normal((4, n + 3))).astype(np.float32)
    sd, dd = U.Dev(src), U.Dev(nbytes=4 * 4 * (2 * n))
    L.check(lib.pi_op_copy_rows(sd.ptr, n + 3, dd.ptr + 4 * n, 2 * n, n, 4, None))
    assert np.array_equal(dd.get(np.float32, (4, 2 * n))[:, n:], src[:, :n]) and not dd.get(np.float32, (4, 2 * n))[:, :n].any()


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,R,mode", [(3, 1, 8, 6, 4, "window"), (4, 4, 70, 66, 70, "gated"), (2, 1, 5, 130, 0, "window"), (6, 2, 88, 10, 44, "gated"), (2, 2, 12, 4, 12, "window")])
def test_queries_and_keys_for_both_mixers(H, G, D, V, R, mode):
    """window kind: norm with a shared weight, then halves (i, i + R/2) turned; gated kind: neighbours (2i, 2i + 1) turned by stretched steps, no norm; values cached as they are; the rest of a head untouched"""
    U, lib = gpu()
    rng = np.random.default_rng(H * D + R)
    T, n_ctx, eps = 5, 40, 1e-5
    stride = H * D + G * D + G * V + 3
    qkv = rng.standard_normal((T, stride)).astype(np.float32)
    qw, kw = rng.standard_normal(D).astype(np.float32), rng.standard_normal(D).astype(np.float32)
    pos = np.array([0, 1, 17, 30, 39], np.int32)
    cells = np.array([7, 8, 9, 10, 11], np.int32)
    rot = {"dims": R, "base": 50.0}
    if mode == "gated" and R:
        rot["scaling"] = {"factor": 3.0, "low": 0.5, "high": 4.0, "original": 20}
    sc = rot.get("scaling")
    table = lib.pi_rotary_table_create_scaled(48, R, 50.0, sc["factor"] if sc else 1.0, sc["low"] if sc else 1.0, sc["high"] if sc else 1.0, sc["original"] if sc else 0)
    assert table
    xd, qwd, kwd, pd = U.Dev(qkv), U.Dev(qw), U.Dev(kw), U.Dev(pos)
    qo, kc, vc, cp = U.Dev(nbytes=4 * T * H * D), U.Dev(nbytes=4 * n_ctx * G * D), U.Dev(nbytes=4 * n_ctx * G * V), U.Dev(nbytes=4 * n_ctx)
    dyn = U.Dev(np.array([7, 12, T, 0], np.int32))
    base = xd.ptr
    L.check(lib.pi_op_qkv_prepare_ex(base, base + 4 * H * D, base + 4 * (H * D + G * D), stride, qwd.ptr if mode == "window" else None, kwd.ptr if mode == "window" else None, eps, H, G, D, V, table,
                                     NORM_FIRST if mode == "window" else NORM_NONE, HALVES if mode == "window" else NEIGHBOURS, 0, pd.ptr, T, qo.ptr, H * D, kc.ptr, vc.ptr, cp.ptr, dyn.ptr, None))
    got_q, got_k, got_v = qo.get(np.float32, (T, H, D)), kc.get(np.float32, (n_ctx, G, D)), vc.get(np.float32, (n_ctx, G, V))
    for t in range(T):
        q = qkv[t, :H * D].astype(np.float64).reshape(H, D)
        k = qkv[t, H * D:H * D + G * D].astype(np.float64).reshape(G, D)
        v = qkv[t, H * D + G * D:H * D + G * D + G * V].reshape(G, V)
        prep = (lambda y, w: O.rotate(O.unit_rms(y, eps) * w, int(pos[t]), rot if R else None, False)) if mode == "window" else (lambda y, w: O.rotate(y, int(pos[t]), rot if R else None, True))
        assert rel_rms(got_q[t], np.stack([prep(q[h], qw) for h in range(H)])) < 3e-6
        assert rel_rms(got_k[cells[t]], np.stack([prep(k[g], kw) for g in range(G)])) < 3e-6
        assert np.array_equal(got_v[cells[t]], v)
    assert np.array_equal(cp.get(np.int32)[7:12], pos)
    lib.pi_rotary_table_free(table)


def window_attention_ref(q, kc, vc, cpos, vis, pos, scale, size, pool, sink, gate, H, G, n_ctx):
    """explicit sums over a cache whose rows n_ctx + c hold the pooled block that cell c closes"""
    T, V = q.shape[0], vc.shape[2]
    out = np.zeros((T, H, V))
    for t in range(T):
        rows = []
        for c in range(vis.shape[1]):
            if not vis[t, c]:
                continue
            d = pos[t] - cpos[c]
            if not size or d < size:
                rows.append(c)
            elif pool and (cpos[c] + 1) % pool == 0:
                rows.append(n_ctx + c)
        for h in range(H):
            g = h // (H // G)
            s = np.array([q[t, h].astype(np.float64) @ kc[r, g] for r in rows]) * scale
            w = O.softmax_with(s, None if sink is None else float(sink[h])) if len(rows) else []
            for wi, r in zip(w, rows):
                out[t, h] += wi * vc[r, g]
            if gate is not None:
                out[t, h] *= O.sigmoid(gate[t, h])
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,size,pool,n_kv,T", [(1, 1, 4, 6, 3, 2, 20, 2), (3, 1, 8, 6, 7, 3, 70, 5), (8, 2, 80, 72, 48, 16, 700, 9), (4, 4, 33, 130, 100, 0, 300, 4), (12, 2, 16, 24, 0, 0, 520, 3),
                                                       (2, 2, 64, 64, 300, 7, 1100, 2), (4, 2, 96, 64, 9, 64, 400, 6)])
@pytest.mark.parametrize("kind", ["sink", "gate"])
@pytest.mark.parametrize("splits", [False, True])
def test_window_attention_against_explicit_sums(H, G, D, V, size, pool, n_kv, T, kind, splits):
    """cells in any order, garbage behind the live cells and in the pooled rows nobody may read, large scores (the running maximum matters); a learned sink, or a plain soft-max with a gate per head;
    in one launch, and with the cell range cut into splits that a second launch merges (scratch given: passes of few tokens take that path)"""
    U, lib = gpu()
    rng = np.random.default_rng(H + D + n_kv)
    n_ctx = n_kv + 13
    if kind == "gate":
        pool = 0
    kc, vc = (rng.standard_normal((2 * n_ctx, G, D)) * 1.5).astype(np.float32), rng.standard_normal((2 * n_ctx, G, V)).astype(np.float32)
    cpos = rng.permutation(n_ctx).astype(np.int32)
    kc[n_kv:n_ctx], vc[n_kv:n_ctx] = np.nan, np.nan
    for c in range(n_ctx):                                            # pooled rows exist on cells that close a block only
        if not pool or (cpos[c] + 1) % pool or c >= n_kv:
            kc[n_ctx + c], vc[n_ctx + c] = np.nan, np.nan
    pos = np.sort(rng.integers(n_kv // 2, n_kv, T)).astype(np.int32)
    vis = (cpos[None, :n_kv] <= pos[:, None]) & (rng.random((T, n_kv)) < 0.8)
    for t in range(T):                                               # (the mask never shows a later position; a token sees at least itself)
        own = np.nonzero(cpos[:n_kv] <= pos[t])[0]
        vis[t, own[np.argmax(cpos[own])]] = True
    q = (rng.standard_normal((T, H, D)) * 2).astype(np.float32)
    sink = rng.standard_normal(H).astype(np.float32) * 2 if kind == "sink" else None
    gate = rng.standard_normal((T, H + 2)).astype(np.float32) if kind == "gate" else None
    qd, kd, vd, cd, md, pd = U.Dev(q), U.Dev(kc), U.Dev(vc), U.Dev(cpos), U.Dev(pack_mask(vis, n_kv)), U.Dev(pos)
    sd, gd = (U.Dev(sink) if sink is not None else None), (U.Dev(gate) if gate is not None else None)
    od, dyn = U.Dev(nbytes=4 * T * H * V), U.Dev(np.array([0, n_kv, T, 0], np.int32))
    n_scr = lib.pi_op_window_attention_scratch_floats(H, V, T) if splits else 0
    scr = U.Dev(np.full(max(n_scr, 1), np.nan, np.float32))
    L.check(lib.pi_op_window_attention(qd.ptr, H * D, kd.ptr, vd.ptr, cd.ptr, md.ptr, pd.ptr, None, sd.ptr if sd else None, gd.ptr if gd else None, H + 2, SIGMOID, 0.6, 1.0, SOFTMAX, 0.0, WINDOW, size,
                                       pool if size else 0, n_ctx, 0, H, G, D, V, T, n_kv, scr.ptr if splits else None, n_scr, od.ptr, H * V, dyn.ptr, None))
    want = window_attention_ref(q, kc.astype(np.float64), vc.astype(np.float64), cpos, vis, pos, 0.6, size, pool if size else 0, sink, gate[:, :H] if gate is not None else None, H, G, n_ctx)
    assert rel_rms(od.get(np.float32, (T, H, V)), want) < 5e-6


@pytest.mark.gpu
@pytest.mark.parametrize("G,D,V,pool,n_tok,here", [(1, 4, 6, 3, 7, False), (2, 80, 72, 16, 40, False), (3, 33, 130, 5, 4, True), (2, 8, 8, 1, 3, True), (1, 16, 300, 64, 1, True), (2, 96, 64, 8, 70, False)])
def test_pooled_rows_are_the_means_of_their_blocks(G, D, V, pool, n_tok, here):
    """a pass whose tokens close blocks that began in earlier passes (cells anywhere in the table) and inside the pass; position order of the sum; rows of tokens that close nothing stay untouched;
    through the operator of its own and through the attention launch's extra workgroups"""
    U, lib = gpu()
    rng = np.random.default_rng(D + pool)
    first = 2 * pool + 1 if pool > 1 else 5                          # the pass starts inside a block
    n_kv = first + n_tok + 9
    n_ctx = n_kv + 4
    kc, vc = rng.standard_normal((2 * n_ctx, G, D)).astype(np.float32), rng.standard_normal((2 * n_ctx, G, V)).astype(np.float32)
    head = int(rng.integers(0, n_kv - n_tok))
    old = [c for c in rng.permutation(n_kv) if not head <= c < head + n_tok][:first]      # earlier positions sit anywhere in the table, the pass's own cells are consecutive
    cell_of = np.array(old + list(range(head, head + n_tok)), np.int32)
    cpos = np.full(n_ctx, 10 ** 6, np.int32)
    cpos[cell_of] = np.arange(first + n_tok)
    pos = np.arange(first, first + n_tok).astype(np.int32)
    vis = (cpos[None, :n_kv] <= pos[:, None])
    other = [c for c in range(n_kv) if cpos[c] == 10 ** 6]           # another sequence's cells at the same positions: never shown by the mask
    cpos[other] = rng.integers(0, first + n_tok, len(other))
    before_k, before_v = kc.copy(), vc.copy()
    kd, vd, cd, md, pd, dyn = U.Dev(kc), U.Dev(vc), U.Dev(cpos), U.Dev(pack_mask(vis, n_kv)), U.Dev(pos), U.Dev(np.array([head, n_kv, n_tok, 0], np.int32))
    if here:
        H = 2 * G
        q, od = U.Dev(rng.standard_normal((n_tok, H * D)).astype(np.float32)), U.Dev(nbytes=4 * n_tok * H * V)
        n_scr = lib.pi_op_window_attention_scratch_floats(H, V, n_tok)
        scr = U.Dev(nbytes=4 * n_scr)                                 # (with scratch: the pooling workgroups sit behind the cell splits' in the launch)
        L.check(lib.pi_op_window_attention(q.ptr, H * D, kd.ptr, vd.ptr, cd.ptr, md.ptr, pd.ptr, None, None, None, 0, NONE, 0.1, 1.0, SOFTMAX, 0.0, WINDOW, max(n_tok, 2), pool, n_ctx, 1, H, G, D, V, n_tok, n_kv,
                                           scr.ptr, n_scr, od.ptr, H * V, dyn.ptr, None))
    else:
        L.check(lib.pi_op_pool_blocks(kd.ptr, vd.ptr, cd.ptr, md.ptr, pd.ptr, pool, n_ctx, G, D, V, n_tok, n_kv, dyn.ptr, None))
    got_k, got_v = kd.get(np.float32, (2 * n_ctx, G, D)), vd.get(np.float32, (2 * n_ctx, G, V))
    closed = 0
    for t in range(n_tok):
        row = n_ctx + head + t
        if (pos[t] + 1) % pool:
            assert np.array_equal(got_k[row], before_k[row]) and np.array_equal(got_v[row], before_v[row])
            continue
        members = cell_of[pos[t] - pool + 1:pos[t] + 1]
        assert rel_rms(got_k[row], before_k[members].astype(np.float64).mean(0)) < 1e-6 and rel_rms(got_v[row], before_v[members].astype(np.float64).mean(0)) < 1e-6
        closed += 1
    assert closed >= (1 if n_tok >= pool else 0) and np.array_equal(got_k[:n_ctx], before_k[:n_ctx])


@pytest.mark.gpu
@pytest.mark.parametrize("size,pool,p", [(8, 4, 23), (64, 8, 200), (5, 3, 11), (300, 16, 700), (40, 40, 119), (1, 1, 6)])
def test_window_and_block_edges_and_the_sink(size, pool, p):
    """one made key far louder than every other: on the window's first position it takes the mass; one position earlier it counts only through its block's mean — and not at all while that
    block has not wholly left the window; a huge sink takes everything"""
    U, lib = gpu()
    rng = np.random.default_rng(size + p)
    D, V, n_kv = 8, 5, p + 1
    n_ctx = n_kv + 3
    kc, vc = np.zeros((2 * n_ctx, 1, D), np.float32), np.zeros((2 * n_ctx, 1, V), np.float32)
    kc[:n_kv], vc[:n_kv] = rng.standard_normal((n_kv, 1, D)) * 0.1, rng.standard_normal((n_kv, 1, V))
    cpos = np.arange(n_ctx).astype(np.int32)
    q = np.zeros((1, D), np.float32)
    q[0, 0] = 1.0
    vis = np.ones((1, n_kv), bool)

    def run(loud, sink_value):
        k2, v2 = kc.copy(), vc.copy()
        k2[loud, 0, 0] = 60.0 * pool
        for b in range(n_kv // pool):                                # pooled rows as the pooling operator leaves them
            k2[n_ctx + b * pool + pool - 1], v2[n_ctx + b * pool + pool - 1] = k2[b * pool:(b + 1) * pool].mean(0), v2[b * pool:(b + 1) * pool].mean(0)
        ds = [U.Dev(a) for a in (q, k2, v2, cpos, pack_mask(vis, n_kv), np.array([p], np.int32), np.array([sink_value], np.float32), np.array([0, n_kv, 1, 0], np.int32))]
        od = U.Dev(nbytes=4 * V)
        n_scr = lib.pi_op_window_attention_scratch_floats(1, V, 1)
        scr = U.Dev(nbytes=4 * n_scr)
        L.check(lib.pi_op_window_attention(ds[0].ptr, D, ds[1].ptr, ds[2].ptr, ds[3].ptr, ds[4].ptr, ds[5].ptr, None, ds[6].ptr, None, 0, NONE, 1.0, 1.0, SOFTMAX, 0.0, WINDOW, size, pool, n_ctx, 0, 1, 1, D, V, 1, n_kv,
                                           scr.ptr, n_scr, od.ptr, V, ds[7].ptr, None))
        return od.get(np.float32, (V,)).astype(np.float64), v2

    edge = p - size + 1                                               # the window's first position
    got, v2 = run(edge, 0.0)
    assert np.allclose(got, v2[edge, 0], atol=1e-5)                   # just inside: the loud key itself
    if edge >= 1:
        out_pos = edge - 1
        b = out_pos // pool
        got, v2 = run(out_pos, 0.0)
        if b * pool + pool - 1 <= p - size:                           # its block lies wholly behind the window: the block's mean value, carried by a mean key that is still loud
            assert np.allclose(got, v2[n_ctx + b * pool + pool - 1, 0], atol=1e-5)
        else:                                                         # not yet: nobody sees the key, the output is an ordinary mixture
            quiet, _ = run(n_kv + 1, 0.0)
            assert np.allclose(got, quiet, atol=1e-5)
    got, _ = run(edge, 1e4)
    assert np.abs(got).max() < 1e-20                                  # the sink has no value


@pytest.mark.gpu
def test_a_far_block_among_hundreds_is_heard():
    """1500 positions, windows of 32, blocks of 8: one far block's keys are made loud; the token's output is that block's mean value, at every distance behind the window"""
    U, lib = gpu()
    rng = np.random.default_rng(5)
    D, V, size, pool, n_kv = 16, 12, 32, 8, 1500
    n_ctx = n_kv
    kc, vc = np.zeros((2 * n_ctx, 2, D), np.float32), np.zeros((2 * n_ctx, 2, V), np.float32)
    kc[:n_kv], vc[:n_kv] = rng.standard_normal((n_kv, 2, D)) * 0.1, rng.standard_normal((n_kv, 2, V))
    cpos = rng.permutation(n_ctx).astype(np.int32)
    cell_at = np.argsort(cpos)
    for block in (0, 7, 100, 182):
        k2, v2 = kc.copy(), vc.copy()
        k2[cell_at[block * pool:(block + 1) * pool], 1, 3] = 40.0
        kd, vd, cd = U.Dev(k2), U.Dev(v2), U.Dev(cpos)
        for t0 in range(0, n_kv, 300):                               # pooled rows through the operator, pass by pass, as the engine would write them
            n = min(300, n_kv - t0)
            pos = np.arange(t0, t0 + n).astype(np.int32)
            vis = cpos[None, :] <= pos[:, None]
            dyn = np.concatenate([[0, n_kv, n, 1], cell_at[t0:t0 + n], np.full(n, n_kv)]).astype(np.int32)
            md, pd, dd = U.Dev(pack_mask(vis, n_kv)), U.Dev(pos), U.Dev(dyn)
            L.check(lib.pi_op_pool_blocks(kd.ptr, vd.ptr, cd.ptr, md.ptr, pd.ptr, pool, n_ctx, 2, D, V, n, n_kv, dd.ptr, None))
            L.check(lib.pi_stream_sync(None))
        q = np.zeros((1, 4, D), np.float32)
        q[0, :, 3] = 1.0
        p = n_kv - 1
        vis = np.ones((1, n_kv), bool)
        od = U.Dev(nbytes=4 * 4 * V)
        qd, md, pd, dd = U.Dev(q), U.Dev(pack_mask(vis, n_kv)), U.Dev(np.array([p], np.int32)), U.Dev(np.array([0, n_kv, 1, 0], np.int32))
        n_scr = lib.pi_op_window_attention_scratch_floats(4, V, 1)
        scr = U.Dev(nbytes=4 * n_scr)
        L.check(lib.pi_op_window_attention(qd.ptr, 4 * D, kd.ptr, vd.ptr, cd.ptr, md.ptr, pd.ptr, None, None, None, 0, NONE, 1.0, 1.0, SOFTMAX, 0.0, WINDOW, size, pool,
                                           n_ctx, 0, 4, 2, D, V, 1, n_kv, scr.ptr, n_scr, od.ptr, 4 * V, dd.ptr, None))
        got = od.get(np.float32, (4, V))
        mean_v = v2[cell_at[block * pool:(block + 1) * pool], 1].astype(np.float64).mean(0)
        assert np.allclose(got[2], mean_v, atol=1e-5) and np.allclose(got[3], mean_v, atol=1e-5)         # the heads of key head 1
        assert not np.allclose(got[0], mean_v, atol=1e-2)                                                 # key head 0 hears nothing special


@pytest.mark.gpu
@pytest.mark.parametrize("n_out,top", [(5, 2), (8, 8), (70, 4), (1, 1), (3, 1)])
@pytest.mark.parametrize("exact", [1, 0])
def test_router_takes_the_largest_logits(n_out, top, exact):
    """logit + bias; the chosen in falling order, the lower index on a tie; weights over the chosen alone"""
    U, lib = gpu()
    rng = np.random.default_rng(n_out * 10 + top)
    K, T = 48, 9
    Wr = O.bf16_round(rng.standard_normal((n_out, K)).astype(np.float32))
    bias = rng.standard_normal(n_out).astype(np.float32)
    x = O.bf16_round(rng.standard_normal((T, K)).astype(np.float32))
    if n_out >= 3:
        Wr[2], bias[2] = Wr[0], bias[0]                                # a tie between outputs 0 and 2
    w, xd, bd = upload_bf16(lib, Wr), U.Dev(x), U.Dev(bias)
    sel, selw = U.Dev(nbytes=4 * T * top), U.Dev(nbytes=4 * T * top)
    L.check(lib.pi_op_moe_route_top_logits(w, bd.ptr, xd.ptr, K, T, top, exact, sel.ptr, selw.ptr, None))
    got_s, got_w = sel.get(np.int32, (T, top)), selw.get(np.float32, (T, top))
    for t in range(T):
        chosen, weights = O.route({"router": Wr.astype(np.float64), "router.b": bias.astype(np.float64)}, "", top, x[t].astype(np.float64))
        assert list(got_s[t]) == chosen and rel_rms(got_w[t], weights) < 1e-5
    lib.pi_weight_free(w)


@pytest.mark.gpu
@pytest.mark.parametrize("E,ff,K,T,top,limit", [(5, 6, 40, 3, 2, 1.25), (8, 64, 128, 70, 3, 0.8), (1, 1, 8, 2, 1, 0.0), (6, 24, 64, 40, 6, 2.0)])
@pytest.mark.parametrize("exact", [1, 0])
def test_clipped_experts_through_both_paths(E, ff, K, T, top, limit, exact):
    """gathered mat-vecs (few tokens, fp32) and the grouped matrix-core path (many): the gate bounded from above, the other half on both sides, (u + 1), weights from the router's slots"""
    U, lib = gpu()
    rng = np.random.default_rng(E + ff + T)
    up = O.bf16_round((rng.standard_normal((E, 2 * ff, K)) * 3 / np.sqrt(K)).astype(np.float32))
    down = O.bf16_round((rng.standard_normal((E, K, ff)) / np.sqrt(ff)).astype(np.float32))
    x = O.bf16_round(rng.standard_normal((T, K)).astype(np.float32))
    sel = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    selw = rng.uniform(0.1, 1.0, (T, top)).astype(np.float32)
    wu, wd = upload_bf16(lib, up.reshape(E * 2 * ff, K)), upload_bf16(lib, down.reshape(E * K, ff))
    xd, sd, swd, od = U.Dev(x), U.Dev(sel), U.Dev(selw), U.Dev(nbytes=4 * T * K)
    upd, dnd = U.Dev(nbytes=4 * T * top * 2 * ff), U.Dev(nbytes=4 * T * top * K)
    grouped = lib.pi_op_moe_grouped_ok(wu, wd, E, ff, GLU_CLIPPED, T, top, exact)
    if grouped:
        idx = U.Dev(nbytes=4 * lib.pi_op_moe_grouped_index_ints(T, top, E))
        L.check(lib.pi_op_moe_experts_grouped_glu(wu, wd, E, ff, GLU_CLIPPED, limit, xd.ptr, K, sd.ptr, swd.ptr, T, top, upd.ptr, dnd.ptr, idx.ptr, od.ptr, K, None))
    else:
        L.check(lib.pi_op_moe_experts_glu(wu, wd, E, ff, GLU_CLIPPED, limit, xd.ptr, K, sd.ptr, swd.ptr, T, top, exact, upd.ptr, od.ptr, K, None))
    want = np.zeros((T, K))
    for t in range(T):
        for e, wgt in zip(sel[t], selw[t]):
            Tn = {"gate": up[e, :ff].astype(np.float64), "up": up[e, ff:].astype(np.float64), "down": down[e].astype(np.float64)}
            want[t] += wgt * O.clipped_expert(Tn, "", limit if limit > 0 else None, x[t].astype(np.float64))
    assert rel_rms(od.get(np.float32, (T, K)), want) < (3e-6 if exact else 1e-2)
    assert (grouped != 0) == (not exact and T * top >= 32 and ff % 8 == 0)
    lib.pi_weight_free(wu)
    lib.pi_weight_free(wd)


@pytest.mark.gpu
@pytest.mark.parametrize("ff,limit,gated", [(7, 0.75, True), (300, 0.0, True), (40, 1.5, False)])
def test_gated_product_of_the_shared_expert(ff, limit, gated):
    U, lib = gpu()
    rng = np.random.default_rng(ff)
    T, stride = 6, 2 * ff + 3
    x = (rng.standard_normal((T, stride)) * 2).astype(np.float32)
    xd, od = U.Dev(x), U.Dev(nbytes=4 * T * (ff + 1))
    L.check(lib.pi_op_glu_mul_ex(xd.ptr, stride, ff, GLU_CLIPPED, limit, 2 * ff if gated else -1, T, od.ptr, ff + 1, None))
    g, u = x[:, :ff].astype(np.float64), x[:, ff:2 * ff].astype(np.float64)
    if limit > 0:
        g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
    want = g * O.sigmoid(1.702 * g) * (u + 1.0) * (O.sigmoid(x[:, 2 * ff:2 * ff + 1].astype(np.float64)) if gated else 1.0)
    assert rel_rms(od.get(np.float32, (T, ff + 1))[:, :ff], want) < 3e-6
    L.check(lib.pi_op_glu_mul_ex(xd.ptr, stride, ff, GLU_SILU, 0.0, -1, T, od.ptr, ff + 1, None))
    assert rel_rms(od.get(np.float32, (T, ff + 1))[:, :ff], x[:, :ff].astype(np.float64) * O.sigmoid(x[:, :ff].astype(np.float64)) * x[:, ff:2 * ff]) < 3e-6


@pytest.mark.gpu
@pytest.mark.parametrize("taps", [1, 3, 11])
def test_convolution_without_activation_over_three_tables(taps):
    """q | k | v channels side by side, no bias, no activation; sequences that start, continue across passes with fewer tokens than taps, and passes above 32 tokens"""
    U, lib = gpu()
    rng = np.random.default_rng(taps)
    ch, slots = 37, 2
    w = rng.standard_normal((ch, taps)).astype(np.float32)
    wd = U.Dev(w)
    state = U.Dev((rng.standard_normal((slots, max(taps - 1, 1), ch)) * 30).astype(np.float32))
    windows = {}
    for step in ([(1, 2, True)], [(1, 1, False), (0, 4, True)], [(0, 45, False), (1, 3, False)], [(1, 1, False)]):
        T = sum(c for _, c, _ in step)
        x = rng.standard_normal((T, ch + 2)).astype(np.float32)
        rec, want, at = [], np.zeros((T, ch)), 0
        for slot, count, fresh in step:
            if fresh:
                windows[slot] = [np.zeros(ch) for _ in range(taps - 1)]
            for i in range(count):
                rec.append(slot | (F if fresh and i == 0 else 0))
                want[at], windows[slot] = O.short_conv(w.astype(np.float64), windows[slot], x[at, :ch].astype(np.float64))
                at += 1
        od, xd, rd = U.Dev(nbytes=4 * T * ch), U.Dev(x), U.Dev(np.array(rec, np.int32))
        L.check(lib.pi_op_causal_conv(xd.ptr, ch + 2, ch, taps, wd.ptr, None, state.ptr, rd.ptr, T, NONE, od.ptr, ch, None))
        assert rel_rms(od.get(np.float32, (T, ch)), want) < 2e-6


# ---- whole models through llama_decode ---------------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("exact", [True, False])
def test_prompt_portions_and_decoding_agree_with_the_oracle(tmp_path, variant, exact):
    m = variant_model(variant)
    rng = np.random.default_rng(5)
    toks = [int(t) for t in rng.integers(0, VOCAB, 75)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=96, n_batch=48, exact=exact)
    tol = TOL[exact] * (3 if variant == "wide_heads" else 1)
    whole = np.concatenate([e.ctx.feed(toks[:48], 0, 0), e.ctx.feed(toks[48:], 48, 0)])
    assert within(logit_err(whole, want), exact, tol)
    e.ctx.seq_rm(0, -1, -1)
    parts, at = [], 0
    for n in [2, 3, 31, 2, 1, 1, 7, 2, 5, 1, 1, 1, 2, 16]:                 # portions down to two tokens and single tokens, cut inside windows, blocks and convolution windows
        parts.append(e.ctx.feed(toks[at:at + n], at, 1))
        at += n
    assert at == 75 and within(logit_err(np.concatenate(parts), want), exact, tol)
    e.ctx.seq_rm(1, -1, -1)
    single = np.concatenate([e.ctx.feed(toks[i:i + 1], i, 2) for i in range(40)])
    assert within(logit_err(single, want[:40]), exact, tol)
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_a_wider_model_with_long_passes(tmp_path, exact):
    """widths and passes that reach the matrix-core products and the grouped experts: 300 tokens in passes of 128 (longer than either window), then single tokens"""
    layers = [O.window_layer(heads=4, kv_heads=2, dim=64, vdim=32, conv=4, size=100, pool=16, rot_dims=16, scale=0.2, mlp=O.routed_mlp(experts=8, top=2, ff=64, limit=1.5, shared_ff=96, shared_limit=1.0)),
              O.gated_layer(heads=8, kv_heads=2, dim=32, vdim=48, size=70, rot_dims=32, scale=0.2, scaling=(4.0, 1.0, 4.0, 128), mlp=O.dense_mlp(256))]
    m = small_model(seed=13, layers=layers, width=128, vocab=200, loop=(0, 2, 2))
    rng = np.random.default_rng(6)
    toks = [int(t) for t in rng.integers(0, 200, 320)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=330, n_batch=128, exact=exact)
    got = np.concatenate([e.ctx.feed(toks[:300], 0, 0)] + [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(300, 320)])
    assert within(logit_err(got, want), exact, TOL[exact] * 2)
    e.close()


@pytest.mark.gpu
def test_residual_stream_run_by_run(tmp_path):
    """models cut after 1, 2, ... layers, with and without the repeated run, give the oracle's logits, so the first wrong layer would be named"""
    full = small_model(seed=4)
    toks = [5, 17, 3, 80, 0, 41, 41, 7, 9, 9, 30, 2, 2, 61, 8, 8, 8, 12, 70, 3, 3, 44]
    for n in range(1, 5):
        for loop in (None, {"start": 0, "stop": n, "times": 2}, {"start": n - 1, "stop": n, "times": 3}):
            cfg = dict(full["config"], layers=full["config"]["layers"][:n])
            cfg.pop("loop", None)
            if loop:
                cfg["loop"] = loop
            m = {"config": cfg, "tensors": full["tensors"]}
            e = Engine(tmp_path, m, n_ctx=32, n_batch=8, name="cut%d_%s" % (n, loop and loop["start"]))
            assert logit_err(e.ctx.feed(toks, 0, 0), O.run(m, toks)).max() < TOL[True], (n, loop)
            e.close()


@pytest.mark.gpu
def test_first_tokens_of_a_sequence(tmp_path):
    """a sequence's first tokens see no shifted token, no convolution input and no key of whoever held the slot and the cells before"""
    m = small_model(seed=17)
    e = Engine(tmp_path, m, n_ctx=64, n_batch=8, slots=1)
    for toks in ([7], [7, 7], [80, 7, 3], [3, 80, 7, 7, 2, 2, 2, 9, 1, 4, 4]):
        got = np.concatenate([e.ctx.feed(toks[i:i + 3], i, 0) for i in range(0, len(toks), 3)])
        assert logit_err(got, O.run(m, toks)).max() < TOL[True], toks
        e.ctx.seq_rm(0, -1, -1)
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_batches_of_unequal_requests_equal_each_alone(tmp_path, exact):
    """three requests of unequal length share passes, one starts in the middle: every row equals the same request fed alone through the engine, and in fp32 the oracle"""
    m = small_model(seed=21)
    rng = np.random.default_rng(8)
    reqs = [[int(t) for t in rng.integers(0, VOCAB, n)] for n in (23, 5, 14)]
    extra = [int(t) for t in rng.integers(0, VOCAB, 6)]
    e = Engine(tmp_path, m, n_ctx=128, n_batch=64, exact=exact, slots=5)
    alone = []
    for r in reqs + [extra]:
        alone.append(e.ctx.feed(r, 0, 4))
        e.ctx.seq_rm(4, -1, -1)
    first = [9, 2, 14]
    toks = sum((r[:n] for r, n in zip(reqs, first)), [])
    pos = sum((list(range(n)) for n in first), [])
    seqs = sum(([[s]] * n for s, n in enumerate(first)), [])
    lg = e.ctx.decode(toks, pos, seqs)
    at, got = 0, [[], [], [], []]
    for s, n in enumerate(first):
        got[s].append(lg[at:at + n])
        at += n
    toks = reqs[1][2:] + extra + reqs[0][9:]
    pos = list(range(2, 5)) + list(range(6)) + list(range(9, 23))
    seqs = [[1]] * 3 + [[3]] * 6 + [[0]] * 14
    lg = e.ctx.decode(toks, pos, seqs)
    got[1].append(lg[:3]); got[3].append(lg[3:9]); got[0].append(lg[9:])
    for s, toks in enumerate(reqs + [extra]):
        mine = np.concatenate(got[s])
        assert np.quantile(logit_err(mine, alone[s].astype(np.float64)), 1.0 if exact else 0.9) < (1e-5 if exact else 1e-2), s
        if exact:
            assert logit_err(mine, O.run(m, toks)).max() < TOL[True], s
    e.close()


@pytest.mark.gpu
def test_freed_cells_and_slots_are_used_again(tmp_path):
    """more requests than slots and cells, one after the other and interleaved: a finished request gives back what it held, the next one starts from nothing (no key, no pooled block, no
    convolution input, no shifted token of the earlier owner); a copied sequence continues like the original"""
    m = small_model(seed=31)
    rng = np.random.default_rng(9)
    e = Engine(tmp_path, m, n_ctx=48, n_batch=16, slots=2)
    for round_ in range(5):
        a = [int(t) for t in rng.integers(0, VOCAB, 20 + round_)]
        b = [int(t) for t in rng.integers(0, VOCAB, 11)]
        la = e.ctx.feed(a[:7], 0, 0)
        lb = e.ctx.feed(b, 0, 1)
        la = np.concatenate([la, e.ctx.feed(a[7:], 7, 0)])
        assert e.ctx.state_slots_used() == 2
        with pytest.raises(L.PipeInferError):
            e.ctx.decode([1], [0], [[2]])
        e.ctx.seq_rm(1, -1, -1)
        lc = e.ctx.feed(b[:5], 0, 2)
        for got, toks in ((la, a), (lb, b), (lc, b[:5])):
            assert logit_err(got, O.run(m, toks)).max() < TOL[True], round_
        e.ctx.seq_rm(0, -1, -1)
        e.ctx.seq_rm(2, -1, -1)
        assert e.ctx.state_slots_used() == 0
    a = [int(t) for t in rng.integers(0, VOCAB, 12)]
    e.ctx.feed(a[:8], 0, 0)
    e.ctx.seq_cp(0, 1, -1, -1)
    assert logit_err(e.ctx.feed(a[8:] + [50, 51], 8, 1), O.run(m, a + [50, 51])[8:]).max() < TOL[True]
    assert logit_err(e.ctx.feed(a[8:] + [60], 8, 0), O.run(m, a + [60])[8:]).max() < TOL[True]
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_window_and_block_borders_show_in_prompts_and_in_decoding(tmp_path, exact):
    """sharp attention (a large score scale) over several hundred tokens, windows and blocks that divide neither each other nor the pass width: a key wrongly seen or lost at a window's edge, a
    block seen one token early or late, or a state that forgets, shows far above rounding — the same model with a window one position longer, or blocks one longer, is far away"""
    layers = [O.window_layer(heads=2, kv_heads=1, dim=8, vdim=8, conv=3, size=50, pool=7, rot_dims=4, scale=2.5, mlp=None),
              O.gated_layer(heads=3, kv_heads=3, dim=4, vdim=6, size=37, rot_dims=2, scale=3.0, mlp=O.dense_mlp(16)),
              O.window_layer(heads=2, kv_heads=2, dim=6, vdim=4, conv=2, size=21, pool=30, rot_dims=6, scale=2.0, mlp=None)]
    m = small_model(seed=41, layers=layers, width=32, loop=None)
    rng = np.random.default_rng(12)
    toks = [int(t) for t in rng.integers(0, VOCAB, 330)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=340, n_batch=128, exact=exact)
    got = np.concatenate([e.ctx.feed(toks[:290], 0, 0)] + [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(290, 330)])       # every decoded token moves all three windows; blocks close at 293, 299 (and 300, ...)
    assert within(logit_err(got, want), exact)
    for where, key, value in ((0, "size", 51), (0, "pool", 8), (1, "size", 38), (2, "size", 22)):
        if not exact:
            break                                                     # (at serving precision one key more or less among fifty is not far enough from rounding to tell)
        other = json.loads(json.dumps(m["config"]))
        other["layers"][where]["mixer"]["mask"][key] = value
        off = logit_err(got, O.run({"config": other, "tensors": m["tensors"]}, toks))
        assert off[100:290].max() > 30 * TOL[exact] and off[290:].max() > 30 * TOL[exact], (where, key)      # (far away where the one key more or less carries weight, in the prompt and among the decoded tokens)
    e.close()


@pytest.mark.gpu
def test_long_decoding_token_by_token(tmp_path):
    m = small_model(seed=45)
    rng = np.random.default_rng(13)
    toks = [int(t) for t in rng.integers(0, VOCAB, 200)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=224, n_batch=8, exact=True)
    got = np.concatenate([e.ctx.feed(toks[:3], 0, 0)] + [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(3, 200)])
    assert logit_err(got, want).max() < TOL[True]
    e.close()


@pytest.mark.gpu
def test_greedy_generation_through_the_engine(tmp_path):
    m = small_model(seed=51)
    prompt = [3, 14, 15, 72, 65, 35]
    e = Engine(tmp_path, m, n_ctx=160, n_batch=16, exact=True)
    got = e.ctx.generate(prompt, 100)
    want = O.greedy(m, prompt, 100)
    k = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), len(want))
    if k < len(want):                                               # (an arg-max between two nearly equal logits may fall either way in fp32 against float64: it must be a near tie)
        lg = O.run(m, prompt + want[:k])[-1]
        assert abs(lg[got[k]] - lg[want[k]]) < 1e-3 * np.abs(lg).max()
    assert k >= 20
    e.close()


@pytest.mark.gpu
def test_graph_replays_equal_eager_launches(tmp_path):
    m = small_model(seed=61)
    rng = np.random.default_rng(3)
    toks = [int(t) for t in rng.integers(0, VOCAB, 60)]
    outs = []
    for graphs in (True, False):
        e = Engine(tmp_path, m, n_ctx=64, n_batch=16, exact=False, name="g%d" % graphs)
        e.ctx.set_graphs(graphs)
        lg = []
        for rep in range(3):
            lg.append(np.concatenate([e.ctx.feed(toks[:37], 0, rep % 2), e.ctx.feed(toks[37:38], 37, rep % 2), e.ctx.feed(toks[38:], 38, rep % 2)]))
            e.ctx.seq_rm(rep % 2, -1, -1)
        assert all(np.array_equal(lg[0], x) for x in lg[1:])
        outs.append(lg[0])
        e.close()
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.gpu
def test_generate_command_line(tmp_path, capsys):
    from pipeinfer_amd.tools import generate as G
    m = small_model(seed=71)
    folder = str(tmp_path / "g")
    write(folder, m)
    assert G.main(["--model", folder, "--prompt-ids", "5,6,7", "--n-predict", "12", "--float32"]) == 0
    greedy = [int(t) for t in capsys.readouterr().out.strip().split(",")]
    want = O.greedy(m, [5, 6, 7], 12)
    k = next((i for i, (a, b) in enumerate(zip(greedy, want)) if a != b), 12)
    assert k >= 6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_trace_runner_replays_steps_and_writes_the_wanted_rows(tmp_path, dtype):
    import subprocess
    import sys
    m = variant_model("only_window", seed=81)
    folder, out = str(tmp_path / "model"), str(tmp_path / "out")
    write(folder, m)
    rng = np.random.default_rng(5)
    a, b = [int(t) for t in rng.integers(0, VOCAB, 41)], [int(t) for t in rng.integers(0, VOCAB, 9)]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:3], "want": [0, 2]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[3:33], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[33:40], "want": [6, 1]}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[40:], "want": [0]}], "end": ["a"]},
             {"step": 4, "entries": [{"id": "b", "tokens": b, "want": [8]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out, "--max-tokens", "48", "--n-batch", "16"],
                       input="".join(json.dumps(x) + "\n" for x in steps), capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done %d" % i for i in range(5)]
    la, lb = O.run(m, a), O.run(m, b)
    want = {0: la[[0, 2]], 2: la[[39, 34]], 3: la[[40]], 4: lb[[8]]}
    assert sorted(os.listdir(out)) == sorted("%d.f32" % k for k in want)
    for k, w in want.items():
        got = np.fromfile(os.path.join(out, "%d.f32" % k), "<f4").reshape(-1, VOCAB)
        assert got.shape == w.shape and (logit_err(got, w).max() < TOL[True] if dtype == "float32" else np.median(logit_err(got, w)) < TOL[False]), k
