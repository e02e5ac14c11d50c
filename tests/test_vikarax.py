"""The Vikarax design (a mixer of two parallel branches — chunked attention with sigmoid weights beside a selective recurrence —, layer norms before and after every
sublayer, a learned average over depth, group-limited routing of gated experts) on the engine, held to the plain numpy restatement in tests/vikarax_oracle.py: every
mechanism alone through its operator, then whole models through llama_decode — prompts against token-by-token decoding, portions down to two tokens, batches of unequal
requests, cells and state slots freed and used again, keys at the borders of chunks, long decoding, greedy generation, the trace runner.  Models are small, random and
made here; sizes are chosen so that nothing that could be mixed up is equal."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from pipeinfer_amd import lib as L, llama as LL
from tests import vikarax_oracle as O

BF16 = 30
F = 1 << 30                                    # "this sequence starts from nothing" on the first token of a run (rec words)
SILU, SIGMOID = 1, 2


def bf(rng, *shape, s=1.0):
    return O.bf16_round((rng.standard_normal(shape) * s).astype(np.float32))


def rel_rms(got, want):
    d = np.asarray(got, np.float64) - np.asarray(want, np.float64)
    return float(np.sqrt((d * d).mean()) / (np.sqrt((np.asarray(want, np.float64) ** 2).mean()) + 1e-30))


def logit_err(got, want):
    d = np.asarray(got, np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / (want - want.mean(-1, keepdims=True)).std()


TOL = {True: 3e-4, False: 4e-2}          # exact (fp32) / serving precision (bfloat16 matrix inputs)



def within(err, exact, tol=None):
    """fp32: every position within the tolerance.  Serving precision: a router's near tie (two groups or experts whose scores differ in the third digit) may fall the other way once the
    input is rounded to bfloat16, and that position is then far off although nothing is wrong (with six experts and random routers a few positions in a hundred): most positions must be
    within the tolerance, the fp32 runs of the same tests are the sharp ones"""
    tol = tol if tol is not None else TOL[exact]
    return err.max() < tol if exact else np.quantile(err, 0.85) < tol


ROUTED = O.routed_mlp(6, 2, 10, count=3, keep=2, shared=7)


def small_model(seed=0, width=40, vocab=89, layers=None, **kw):
    rng = np.random.default_rng(seed)
    layers = layers or [O.parallel_layer(mlp=O.dense_mlp(24)),
                        O.parallel_layer(heads=4, kv_heads=2, dim=6, vdim=10, chunk=5, rot_dims=6, r_heads=2, r_vdim=9, state=4, groups=1, conv=4, norm_groups=1, mlp=ROUTED),
                        O.parallel_layer(mlp=None),
                        O.parallel_layer(heads=2, kv_heads=2, dim=10, vdim=4, chunk=16, rot_dims=2, r_heads=3, r_vdim=4, state=7, groups=3, conv=2, norm_groups=3, mlp=ROUTED)]
    return O.random_model(rng, vocab, width, layers, **kw)


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
    assert mod.n_vocab == 89
    buf = C.create_string_buffer(64)
    mod.lib.llama_model_desc.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
    mod.lib.llama_model_desc(mod.h, buf, 64)
    assert buf.value.lower().startswith(b"vikarax")
    mod.free()
    for name, layers in VARIANTS.items():                          # descriptions without chunks, without a rotation, without groups, a shared expert or a feed-forward are read as well
        if layers:
            mv = small_model(seed=1, layers=layers, width=64 if name == "wide_heads" else 40)
            write(str(tmp_path / name), mv)
            LL.Model(str(tmp_path / name)).free()


@pytest.mark.parametrize("breakage", ["type", "kv_heads", "rot", "groups", "keep", "kind", "norm_groups", "left_scale"])
def test_a_wrong_description_is_refused(tmp_path, breakage):
    m = small_model()
    cfg = json.loads(json.dumps(m["config"]))
    if breakage == "type":
        cfg["layers"][0]["type"] = "serial"
    elif breakage == "kv_heads":
        cfg["layers"][1]["mixer"]["left"]["kv_heads"] = 3
    elif breakage == "rot":
        cfg["layers"][0]["mixer"]["left"]["rot"]["dims"] = 5
    elif breakage == "groups":
        cfg["layers"][0]["mixer"]["right"]["groups"] = 3
    elif breakage == "keep":
        cfg["layers"][1]["mlp"]["router"]["groups"]["keep"] = 4
    elif breakage == "kind":
        cfg["layers"][0]["mlp"]["kind"] = "glu"
    elif breakage == "norm_groups":
        cfg["layers"][0]["mixer"]["right"]["norm_groups"] = 3
    elif breakage == "left_scale":
        del cfg["layers"][2]["mixer"]["left_scale"]
    folder = str(tmp_path / "bad")
    O.write_model(folder, cfg, {k: v.astype(np.float32) for k, v in m["tensors"].items()})
    with pytest.raises(L.PipeInferError):
        LL.Model(folder)


def test_oracle_mechanisms_behave_as_stated():
    """the restatement itself: the chunk border, a rotation that keeps lengths and depends on the distance only, a recurrence whose decay of one sums its inputs, the groups of the router"""
    rng = np.random.default_rng(3)
    v = rng.standard_normal(8)
    assert np.isclose(np.linalg.norm(O.rotate(v, 11, 6, 100.0)), np.linalg.norm(v)) and np.array_equal(O.rotate(v, 11, 6, 100.0)[6:], v[6:])
    a, b = rng.standard_normal(4), rng.standard_normal(4)
    assert np.isclose(O.rotate(a, 9, 4, 30.0) @ O.rotate(b, 5, 4, 30.0), O.rotate(a, 104, 4, 30.0) @ O.rotate(b, 100, 4, 30.0))
    m = small_model(seed=3, layers=[O.parallel_layer(chunk=4, mlp=None)])
    T, c = m["tensors"], m["config"]["layers"][0]["mixer"]["left"]
    keys, values = [], []
    hs = rng.standard_normal((6, 40))
    outs = [O.attention_step(T, "l0.mix.left.", c, 1e-5, hs[i], i, keys, values) for i in range(6)]
    alone_k, alone_v = [], []
    O.attention_step(T, "l0.mix.left.", c, 1e-5, hs[3], 3, alone_k, alone_v)                # positions 0..3 are one chunk, 4 starts the next: token 4 sees itself only
    again = O.attention_step(T, "l0.mix.left.", c, 1e-5, hs[4], 4, alone_k, alone_v)
    assert np.allclose(again, outs[4]) and not np.allclose(outs[5], O.attention_step(T, "l0.mix.left.", c, 1e-5, hs[5], 5, [], []))
    mlp = O.routed_mlp(6, 2, 4, count=3, keep=1)
    T = {"r.router": np.eye(6, 8) * np.array([3.0, -9, 2.0, 2.5, 1.0, 1.2])[:, None]}
    idx, w = O.route(T, "r.", mlp, np.ones(8))                                              # group scores: (3, -9) < (2, 2.5): the best single expert loses with its group
    assert idx == [3, 2] and np.allclose(w, O.sigmoid(np.array([2.5, 2.0])))


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
@pytest.mark.parametrize("n", [5, 96, 300, 1000])
def test_layer_norm_of_one_and_of_two_inputs(n):
    U, lib = gpu()
    rng = np.random.default_rng(n)
    T = 4
    a, b, r = ((rng.standard_normal((T, n + 3)) * 3 + 5).astype(np.float32) for _ in range(3))        # (a mean far from zero: the variance must be taken around it)
    w, bias = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    ad, bd, rd, wd, sd, od = U.Dev(a), U.Dev(b), U.Dev(r), U.Dev(w), U.Dev(bias), U.Dev(nbytes=4 * T * n)
    L.check(lib.pi_op_layer_norm_mix(ad.ptr, n + 3, 1.0, None, 0, 0.0, wd.ptr, sd.ptr, 1e-3, n, T, None, 0, od.ptr, n, None))
    want = np.stack([O.layer_norm(a[t, :n].astype(np.float64), w, bias, 1e-3) for t in range(T)])
    assert rel_rms(od.get(np.float32, (T, n)), want) < 2e-6
    L.check(lib.pi_op_layer_norm_mix(ad.ptr, n + 3, 0.8, bd.ptr, n + 3, -1.3, wd.ptr, sd.ptr, 1e-3, n, T, rd.ptr, n + 3, od.ptr, n, None))
    want = np.stack([r[t, :n] + O.layer_norm(0.8 * a[t, :n].astype(np.float64) - 1.3 * b[t, :n], w, bias, 1e-3) for t in range(T)])
    assert rel_rms(od.get(np.float32, (T, n)), want) < 2e-6


@pytest.mark.gpu
@pytest.mark.parametrize("n,J", [(40, 1), (320, 4), (1000, 7)])
def test_block_end_in_one_launch(n, J):
    """post-norm + residual into the history's last entry, the average over the history, the next pre-norm: every stage against the separate formulas, also in place"""
    U, lib = gpu()
    rng = np.random.default_rng(n + J)
    T, rows = 3, 5
    a, b, x = (rng.standard_normal((T, n)).astype(np.float32) for _ in range(3))
    hist = rng.standard_normal((J, rows, n)).astype(np.float32)
    w, wb, w2, w2b = (rng.standard_normal(n).astype(np.float32) for _ in range(4))
    coef = rng.standard_normal(J).astype(np.float32)
    ad, bd, xd, hd, cd, od = U.Dev(a), U.Dev(b), U.Dev(x), U.Dev(hist), U.Dev(coef), U.Dev(nbytes=4 * T * n)
    ws = [U.Dev(v) for v in (w, wb, w2, w2b)]
    y = np.stack([x[t] + O.layer_norm(a[t].astype(np.float64) + b[t], w, wb, 1e-4) for t in range(T)])
    mixed = np.einsum("j,jtn->tn", coef[:J - 1].astype(np.float64), hist[:J - 1, :T]) + coef[J - 1] * y
    nxt = np.stack([O.layer_norm(mixed[t], w2, w2b, 1e-4) for t in range(T)])
    last = hd.ptr + 4 * (J - 1) * rows * n
    L.check(lib.pi_op_norm_chain(ad.ptr, n, 1.0, bd.ptr, n, 1.0, ws[0].ptr, ws[1].ptr, 1e-4, n, T, xd.ptr, n, last, n, hd.ptr, rows * n, J, cd.ptr, xd.ptr, n, ws[2].ptr, ws[3].ptr, od.ptr, n, None))
    h2 = hd.get(np.float32, (J, rows, n))
    assert rel_rms(h2[J - 1, :T], y) < 2e-6 and np.array_equal(h2[:J - 1], hist[:J - 1]) and np.array_equal(h2[J - 1, T:], hist[J - 1, T:])
    assert rel_rms(xd.get(np.float32, (T, n)), mixed) < 3e-6 and rel_rms(od.get(np.float32, (T, n)), nxt) < 5e-6
    # without a history: the residual row is updated in place and normed for the next sublayer
    xd = U.Dev(x)
    L.check(lib.pi_op_norm_chain(ad.ptr, n, 0.5, None, 0, 0.0, ws[0].ptr, ws[1].ptr, 1e-4, n, T, xd.ptr, n, xd.ptr, n, None, 0, 0, None, None, 0, ws[2].ptr, ws[3].ptr, od.ptr, n, None))
    y = np.stack([x[t] + O.layer_norm(0.5 * a[t].astype(np.float64), w, wb, 1e-4) for t in range(T)])
    assert rel_rms(xd.get(np.float32, (T, n)), y) < 2e-6 and rel_rms(od.get(np.float32, (T, n)), np.stack([O.layer_norm(y[t], w2, w2b, 1e-4) for t in range(T)])) < 5e-6


@pytest.mark.gpu
def test_depth_mix_softcap_and_gated_product():
    U, lib = gpu()
    rng = np.random.default_rng(2)
    T, n, J, rows = 3, 70, 5, 8                                   # the history holds `rows` rows per state, only T of them are this pass's
    hist, coef = rng.standard_normal((J, rows, n)).astype(np.float32), rng.standard_normal(J).astype(np.float32)
    hd, cd, od = U.Dev(hist), U.Dev(coef), U.Dev(nbytes=4 * T * n)
    for j in (1, 2, J):
        L.check(lib.pi_op_depth_mix(hd.ptr, rows * n, j, cd.ptr, n, T, od.ptr, n, None))
        assert rel_rms(od.get(np.float32, (T, n)), np.einsum("j,jtn->tn", coef[:j].astype(np.float64), hist[:j, :T])) < 1e-6
    x = (rng.standard_normal(500) * 20).astype(np.float32)
    xd = U.Dev(x)
    L.check(lib.pi_op_softcap(xd.ptr, 500, 7.5, None))
    assert rel_rms(xd.get(np.float32, (500,)), 7.5 * np.tanh(x.astype(np.float64) / 7.5)) < 1e-6
    g = rng.standard_normal((T, 2 * 33 + 1)).astype(np.float32)
    gd, od = U.Dev(g), U.Dev(nbytes=4 * T * 33)
    L.check(lib.pi_op_glu_mul(gd.ptr, 67, 33, T, od.ptr, 33, None))
    assert np.array_equal(od.get(np.float32, (T, 33)), g[:, :33] * g[:, 33:66])


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,R", [(3, 1, 8, 6, 4), (4, 4, 70, 66, 70), (2, 1, 5, 130, 0), (6, 2, 88, 10, 44)])
def test_queries_keys_values_are_normed_rotated_and_stored(H, G, D, V, R):
    U, lib = gpu()
    rng = np.random.default_rng(D + V)
    T, n_ctx, first, stride = 5, 20, 9, H * D + G * (D + V) + 3
    buf = rng.standard_normal((T, stride)).astype(np.float32)
    qw, kw = rng.standard_normal(D).astype(np.float32), rng.standard_normal(D).astype(np.float32)
    pos = np.array([0, 1, 37, 38, 399], np.int32)
    tab = lib.pi_rotary_table_create(400, R, 777.0)
    assert tab and lib.pi_rotary_table_positions(tab) == 400
    bd, qd, kd, pd, dyn = U.Dev(buf), U.Dev(qw), U.Dev(kw), U.Dev(pos), U.Dev(np.array([first, first + T, T, 0], np.int32))
    qo, kc, vc, cp = U.Dev(nbytes=4 * T * H * D), U.Dev(np.zeros((n_ctx, G * D), np.float32)), U.Dev(np.zeros((n_ctx, G * V), np.float32)), U.Dev(np.full(n_ctx, -1, np.int32))
    L.check(lib.pi_op_qkv_prepare(bd.ptr, bd.ptr + 4 * H * D, bd.ptr + 4 * (H * D + G * D), stride, qd.ptr, kd.ptr, 1e-4, H, G, D, V, tab, pd.ptr, T, qo.ptr, H * D, kc.ptr, vc.ptr, cp.ptr, dyn.ptr, None))
    q, k, v, cpos = qo.get(np.float32, (T, H, D)), kc.get(np.float32, (n_ctx, G, D)), vc.get(np.float32, (n_ctx, G, V)), cp.get(np.int32, (n_ctx,))
    b64 = buf.astype(np.float64)
    for t in range(T):
        for h in range(H):
            assert rel_rms(q[t, h], O.rotate(O.unit_rms(b64[t, h * D:(h + 1) * D], 1e-4) * qw, int(pos[t]), R, 777.0)) < 3e-6
        for g in range(G):
            assert rel_rms(k[first + t, g], O.rotate(O.unit_rms(b64[t, H * D + g * D:H * D + (g + 1) * D], 1e-4) * kw, int(pos[t]), R, 777.0)) < 3e-6
            o = H * D + G * D + g * V
            assert rel_rms(v[first + t, g], O.unit_rms(b64[t, o:o + V], 1e-4)) < 3e-6
    assert list(cpos[first:first + T]) == list(pos) and (cpos[:first] == -1).all() and (cpos[first + T:] == -1).all()
    assert not k[:first].any() and not k[first + T:].any() and not v[:first].any()
    lib.pi_rotary_table_free(tab)


def chunk_attention_ref(q, kc, vc, cpos, vis, pos, pb, gate, scale, chunk, H, G):
    T, D, V = q.shape[0], kc.shape[2], vc.shape[2]
    out = np.zeros((T, H, V))
    for t in range(T):
        for c in np.nonzero(vis[t])[0]:
            if chunk and cpos[c] < pos[t] // chunk * chunk:
                continue
            for h in range(H):
                g = h // (H // G)
                out[t, h] += O.sigmoid(q[t, h] @ kc[c, g] * scale + pb[h]) * vc[c, g]
        out[t] *= O.sigmoid(gate[t])[:, None]
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,V,chunk,n_kv,T", [(1, 1, 4, 6, 3, 20, 2), (3, 1, 8, 6, 7, 70, 5), (8, 2, 80, 72, 48, 700, 9), (4, 4, 33, 130, 100, 300, 4), (12, 2, 16, 24, 0, 520, 3), (2, 2, 64, 64, 512, 1100, 2), (40, 1, 8, 130, 9, 90, 3)])
def test_chunk_attention_against_explicit_sums(H, G, D, V, chunk, n_kv, T):
    """cells in any order, garbage behind n_kv and in cells that are not this sequence's; the sum has no soft-max, every visible cell of the token's chunk counts with its own sigmoid"""
    U, lib = gpu()
    rng = np.random.default_rng(n_kv + T)
    n_ctx = n_kv + 13
    kc, vc = rng.standard_normal((n_ctx, G, D)).astype(np.float32), rng.standard_normal((n_ctx, G, V)).astype(np.float32)
    kc[n_kv:], vc[n_kv:] = np.nan, np.nan
    cpos = rng.permutation(n_ctx).astype(np.int32)                 # position of every cell: all different, scattered over the cache
    pos = np.array(sorted(rng.integers(0, n_kv, T)), np.int32)
    q, gate = rng.standard_normal((T, H * D + 2)).astype(np.float32), rng.standard_normal((T, H + 1)).astype(np.float32)
    pb = rng.standard_normal(H).astype(np.float32)
    other = rng.random(n_ctx) < 0.2                                # cells of another sequence: masked, whatever their positions
    vis = (cpos[None, :] <= pos[:, None]) & ~other[None, :]
    vis[:, n_kv:] = False
    kc[:n_kv][other[:n_kv]] = 1e30
    dyn = np.array([0, n_kv, T, 0], np.int32)
    d = [U.Dev(a) for a in (q, kc, vc, cpos, pack_mask(vis, n_ctx), pos, pb, gate, dyn)]
    od = U.Dev(nbytes=4 * T * H * V)
    L.check(lib.pi_op_chunk_attention(d[0].ptr, H * D + 2, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, d[5].ptr, d[6].ptr, d[7].ptr, H + 1, SIGMOID, 0.21, -1.5, chunk, H, G, D, V, T, n_ctx, od.ptr, H * V, d[8].ptr, None))
    got = od.get(np.float32, (T, H, V)) / np.float32(-1.5)          # (the factor on the branch's output)
    want = chunk_attention_ref(q[:, :H * D].reshape(T, H, D).astype(np.float64), np.nan_to_num(kc).astype(np.float64), np.nan_to_num(vc).astype(np.float64), cpos, vis, pos, pb.astype(np.float64),
                               gate[:, :H].astype(np.float64), 0.21, chunk, H, G)
    assert np.isfinite(got).all() and rel_rms(got, want) < 2e-5, rel_rms(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("chunk,p", [(8, 23), (8, 24), (64, 127), (64, 128), (5, 4)])
def test_chunk_border_keys_one_inside_one_outside(chunk, p):
    """every weight is pushed to nearly zero by the head's bias except for two made keys: the first position of the query's chunk (must count) and the position just before it (must
    not); their values are unit vectors, so the output names which keys were seen.  One further key far back in an earlier chunk would win if chunks were forgotten altogether"""
    U, lib = gpu()
    rng = np.random.default_rng(chunk + p)
    H, G, D, V, n_ctx = 2, 1, 16, 8, 160
    kc, vc = (rng.standard_normal((n_ctx, G, D)) * 0.1).astype(np.float32), np.zeros((n_ctx, G, V), np.float32)
    cpos = np.arange(n_ctx, dtype=np.int32)[::-1].copy()           # cell c holds position n_ctx - 1 - c
    cell = lambda position: n_ctx - 1 - position
    q = rng.standard_normal((1, H * D)).astype(np.float32)
    start = p // chunk * chunk
    for position, col in ((start, 0), (start - 1, 1), (0 if start > 1 else -1, 2)):
        if position >= 0:
            kc[cell(position), 0] = q[0, :D] / np.linalg.norm(q[0, :D]) * 40        # score = |q| * 40 * scale: far above the bias
            vc[cell(position), 0, col] += 1.0
    vis = (cpos[None, :] <= p)
    d = [U.Dev(a) for a in (q, kc, vc, cpos, pack_mask(vis, n_ctx), np.array([p], np.int32), np.full(H, -12.0, np.float32), np.array([0, n_ctx, 1, 0], np.int32))]
    od = U.Dev(nbytes=4 * H * V)
    L.check(lib.pi_op_chunk_attention(d[0].ptr, H * D, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, d[5].ptr, d[6].ptr, None, 0, 0, 1.0, 1.0, chunk, H, G, D, V, 1, n_ctx, od.ptr, H * V, d[7].ptr, None))
    got = od.get(np.float32, (H, V))[0]
    assert abs(got[0] - 1.0) < 1e-3 and abs(got[1]) < 1e-3 and abs(got[2]) < 1e-3, got          # the chunk's first position counts; the one before it and the far one do not


def conv_ref(x, w, b, tails, rec, taps):
    """token by token: tails[slot] = the sequence's last taps - 1 inputs"""
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        s = rec[t] & ~F
        if rec[t] & F:
            tails[s] = [np.zeros(x.shape[1]) for _ in range(taps - 1)]
        window = tails[s] + [x[t]]
        out[t] = O.silu(b + sum(w[:, l] * window[l] for l in range(taps)))
        tails[s] = window[1:]
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("taps,channels", [(4, 300), (2, 7), (3, 64), (1, 10), (7, 33), (8, 20), (11, 9)])
@pytest.mark.parametrize("fused", [False, True])
def test_causal_conv_over_sequences_and_passes(taps, channels, fused):
    U, lib = gpu()
    rng = np.random.default_rng(taps * channels)
    slots = 4
    hbv, hav = rng.standard_normal(3).astype(np.float32), rng.standard_normal(3).astype(np.float32)
    hb, ha = U.Dev(hbv), U.Dev(hav)
    w, b = rng.standard_normal((channels, taps)).astype(np.float32), rng.standard_normal(channels).astype(np.float32)
    state = rng.standard_normal((slots, max(taps - 1, 1), channels)).astype(np.float32)          # what earlier owners left
    wd, bd, sd = U.Dev(w), U.Dev(b), U.Dev(state)
    tails = {}

    def run(rec):
        T = len(rec)
        x = rng.standard_normal((T, channels + 2)).astype(np.float32)
        xd, rd, od = U.Dev(x), U.Dev(np.array(rec, np.int32)), U.Dev(nbytes=4 * T * channels)
        if fused:                                                   # the entry the engine uses: one launch for short passes (with the recurrence's step sizes), the two kernels otherwise
            raw = rng.standard_normal((T, 3)).astype(np.float32)
            rawd, dtd, decd = U.Dev(raw), U.Dev(nbytes=4 * T * 3), U.Dev(nbytes=4 * T * 3)
            L.check(lib.pi_op_causal_conv_steps(xd.ptr, channels + 2, channels, taps, wd.ptr, bd.ptr, sd.ptr, rd.ptr, T, SILU, od.ptr, channels, rawd.ptr, 3, hb.ptr, ha.ptr, 3, dtd.ptr, decd.ptr, None))
            dt = O.softplus(raw.astype(np.float64) + hbv)
            assert rel_rms(dtd.get(np.float32, (T, 3)), dt) < 1e-6 and rel_rms(decd.get(np.float32, (T, 3)), np.exp(-np.exp(hav.astype(np.float64)) * dt)) < 1e-6
        else:
            L.check(lib.pi_op_causal_conv(xd.ptr, channels + 2, channels, taps, wd.ptr, bd.ptr, sd.ptr, rd.ptr, T, SILU, od.ptr, channels, None))
        want = conv_ref(x[:, :channels].astype(np.float64), w.astype(np.float64), b.astype(np.float64), tails, rec, taps)
        assert rel_rms(od.get(np.float32, (T, channels)), want) < 2e-6, rec
    run([1 | F] + [1] * 9 + [3 | F] + [0 | F, 0])                   # three sequences start: ten tokens, one token, two tokens
    run([3] + [0] + [1, 1])                                        # ... and go on with fewer tokens than taps: old and new inputs mix in the window
    run([3, 3] + [0] * 12)
    run([0] * 20 + [3] * 25)                                        # more than 32 tokens: the fused entry takes the two-kernel path
    run([1])
    run([1 | F] + [1] * 3 + [3])                                   # slot 1 handed to a new sequence
    if taps > 1:
        st = sd.get(np.float32, (slots, taps - 1, channels))
        for s in (0, 1, 3):
            assert rel_rms(st[s], np.stack(tails[s])) < 1e-6
        assert np.array_equal(st[2], state[2])                      # a slot nobody named is untouched


def ssd_ref(C_, B, x, dt, decay, D, S, heads, groups):
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        for h in range(heads):
            g = h // (heads // groups)
            S[h] = decay[t, h] * S[h] + dt[t, h] * np.outer(B[t, g], x[t, h])
            out[t, h] = S[h].T @ C_[t, g] + D[h] * x[t, h]
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("heads,groups,N,P", [(4, 2, 6, 5), (1, 1, 40, 56), (6, 3, 16, 70), (8, 1, 100, 12), (2, 2, 130, 33), (1, 1, 300, 8)])
def test_selective_recurrence_steps_groups_and_long_passes(heads, groups, N, P):
    """dt and the decays from raw values; then the recurrence with per-token decays, keys scaled by dt, B / C shared inside a group, the skip term; passes longer than the
    32-token pieces (states chained across pieces), several sequences per pass, carried and fresh states"""
    U, lib = gpu()
    rng = np.random.default_rng(heads * N + P)
    slots = 3
    inner, gn = heads * P, groups * N
    stride = inner + 2 * gn + 1
    dt_bias, a_log, D = rng.standard_normal(heads).astype(np.float32), (rng.standard_normal(heads) - 1.0).astype(np.float32), rng.standard_normal(heads).astype(np.float32)
    state = rng.standard_normal((slots, heads, N, P)).astype(np.float32)
    sd, bd, ad, dd = U.Dev(state), U.Dev(dt_bias), U.Dev(a_log), U.Dev(D)
    ref = {}

    def run(rec):
        T = len(rec)
        buf = (rng.standard_normal((T, stride)) * 0.5).astype(np.float32)
        raw = (rng.standard_normal((T, heads + 2)) * 2).astype(np.float32)
        raw[0, 0] = 30.0                                            # softplus of a large value is the value
        xd, rd, rawd = U.Dev(buf), U.Dev(np.array(rec, np.int32)), U.Dev(raw)
        dtd, decd, od = U.Dev(nbytes=4 * T * heads), U.Dev(nbytes=4 * T * heads), U.Dev(nbytes=4 * T * inner)
        L.check(lib.pi_op_ssd_steps(rawd.ptr, heads + 2, bd.ptr, ad.ptr, heads, T, dtd.ptr, decd.ptr, None))
        dt = O.softplus(raw[:, :heads].astype(np.float64) + dt_bias)
        decay = np.exp(-np.exp(a_log.astype(np.float64)) * dt)
        assert rel_rms(dtd.get(np.float32, (T, heads)), dt) < 1e-6 and rel_rms(decd.get(np.float32, (T, heads)), decay) < 1e-6
        nscr = lib.pi_op_linear_attention_scratch_floats(heads, N, P, T, slots)
        scr = U.Dev(nbytes=4 * max(nscr, 4))
        L.check(lib.pi_op_linear_attention_ex(xd.ptr + 4 * (inner + gn), xd.ptr + 4 * inner, xd.ptr, stride, heads, groups, N, P, None, decd.ptr, dtd.ptr, heads, dd.ptr, sd.ptr, rd.ptr, T, slots,
                                              scr.ptr, nscr, od.ptr, inner, None))
        got = od.get(np.float32, (T, heads, P))
        b64 = buf.astype(np.float64)
        x, B, C_ = b64[:, :inner].reshape(T, heads, P), b64[:, inner:inner + gn].reshape(T, groups, N), b64[:, inner + gn:inner + 2 * gn].reshape(T, groups, N)
        t = 0
        while t < T:
            s = rec[t] & ~F
            e = t
            while e < T and (rec[e] & ~F) == s:
                e += 1
            if rec[t] & F:
                ref[s] = np.zeros((heads, N, P))
            want = ssd_ref(C_[t:e], B[t:e], x[t:e], dt[t:e], decay[t:e], D.astype(np.float64), ref[s], heads, groups)
            assert rel_rms(got[t:e], want) < 3e-5, (s, t, e, rel_rms(got[t:e], want))
            t = e
    run([2 | F] + [2] * 11 + [0 | F] + [0] * 2)
    run([0] * 70 + [1 | F] + [1] * 32 + [2] * 33)                   # pieces: 32 + 32 + 6 | 32 + 1 | 32 + 1
    run([2])
    run([1] * 5 + [2] * 2)
    run([0 | F] + [0] * 40)                                         # slot 0 again from nothing
    assert rel_rms(sd.get(np.float32, (slots, heads, N, P))[0], ref[0]) < 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("n,groups", [(12, 3), (176, 2), (70, 1), (520, 4), (6, 6)])
def test_gate_then_norm_in_parts(n, groups):
    U, lib = gpu()
    rng = np.random.default_rng(n)
    T = 3
    y, z, w = rng.standard_normal((T, n + 1)).astype(np.float32), rng.standard_normal((T, n + 5)).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    yd, zd, wd = U.Dev(y), U.Dev(z), U.Dev(w)
    L.check(lib.pi_op_gate_group_norm(yd.ptr, n + 1, zd.ptr, n + 5, wd.ptr, 1e-3, 0.6, n, groups, T, yd.ptr, n + 1, None))     # in place, as the engine calls it
    u = y[:, :n].astype(np.float64) * O.silu(z[:, :n].astype(np.float64))
    want = np.stack([np.concatenate([O.unit_rms(part, 1e-3) for part in u[t].reshape(groups, -1)]) * w * 0.6 for t in range(T)])
    got = yd.get(np.float32, (T, n + 1))
    assert rel_rms(got[:, :n], want) < 2e-6 and np.array_equal(got[:, n], y[:, n])


@pytest.mark.gpu
@pytest.mark.parametrize("E,count,keep,top,ff,width,T", [(6, 3, 2, 2, 10, 40, 5), (18, 3, 1, 4, 48, 96, 7), (4, 1, 1, 4, 8, 33, 3), (8, 8, 3, 1, 16, 48, 4), (12, 4, 4, 5, 24, 64, 40), (70, 7, 2, 6, 8, 40, 3)])
@pytest.mark.parametrize("exact", [True, False])
def test_group_limited_router_and_gated_experts(E, count, keep, top, ff, width, T, exact):
    """choice and weights against the restatement; the experts through the gathered mat-vecs and, for a prompt's worth of slots at serving precision, through the grouped matrix-core path"""
    U, lib = gpu()
    rng = np.random.default_rng(E * 7 + top)
    x = rng.standard_normal((T, width)).astype(np.float32)
    mlp = O.routed_mlp(E, top, ff, count=count, keep=keep)
    tens = {"m.router": bf(rng, E, width, s=0.4).astype(np.float64)}
    for e in range(E):
        for n, shape in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff))):
            tens["m.e%d.%s" % (e, n)] = bf(rng, *shape, s=0.25).astype(np.float64)
    ups = np.concatenate([np.concatenate([tens["m.e%d.gate" % e], tens["m.e%d.up" % e]]) for e in range(E)]).astype(np.float32)
    downs = np.concatenate([tens["m.e%d.down" % e] for e in range(E)]).astype(np.float32)
    rd, ud, dd, xd = upload_bf16(lib, tens["m.router"].astype(np.float32)), upload_bf16(lib, ups), upload_bf16(lib, downs), U.Dev(x)
    sel, selw = U.Dev(nbytes=4 * T * top), U.Dev(nbytes=4 * T * top)
    L.check(lib.pi_op_moe_route_groups(rd, xd.ptr, width, T, top, count, keep, int(exact), sel.ptr, selw.ptr, None))
    gs, gw = sel.get(np.int32, (T, top)), selw.get(np.float32, (T, top))
    xin = x.astype(np.float64) if exact else O.bf16_round(x).astype(np.float64)
    for t in range(T):
        idx, w = O.route(tens, "m.", mlp, xin[t])
        assert list(gs[t]) == idx and np.allclose(gw[t], w, rtol=2e-5), t
    want = np.stack([sum(w * O.gated_expert(tens, "m.e%d." % e, xin[t]) for e, w in zip(gs[t], gw[t].astype(np.float64))) for t in range(T)])
    upb, od = U.Dev(nbytes=4 * T * top * 2 * ff), U.Dev(nbytes=4 * T * width)
    L.check(lib.pi_op_moe_experts_act(ud, dd, E, ff, 1, xd.ptr, width, sel.ptr, selw.ptr, T, top, int(exact), upb.ptr, od.ptr, width, None))
    assert rel_rms(od.get(np.float32, (T, width)), want) < (1e-5 if exact else 6e-3)
    if lib.pi_op_moe_grouped_ok(ud, dd, E, ff, 1, T, top, int(exact)):
        dn, idx_ = U.Dev(nbytes=4 * T * top * width), U.Dev(nbytes=4 * lib.pi_op_moe_grouped_index_ints(T, top, E))
        od2 = U.Dev(nbytes=4 * T * width)
        L.check(lib.pi_op_moe_experts_grouped_act(ud, dd, E, ff, 1, xd.ptr, width, sel.ptr, selw.ptr, T, top, upb.ptr, dn.ptr, idx_.ptr, od2.ptr, width, None))
        assert rel_rms(od2.get(np.float32, (T, width)), want) < 6e-3
    else:
        assert exact or T * top < 32
    for h in (rd, ud, dd):
        lib.pi_weight_free(h)


# ---- whole models through llama_decode ---------------------------------------------------------------------------------------------------
VARIANTS = {
    "mixed": None,
    # values that other models make equal or one: a single head everywhere, as many key heads as query heads, everything rotated / nothing rotated, no chunks, chunks of one
    # position, one group, as many groups as heads, two taps, one tap, top = 1, every group kept, no shared expert, a layer without feed-forward first
    "edges": [O.parallel_layer(heads=1, kv_heads=1, dim=6, vdim=6, chunk=0, rot_dims=6, r_heads=1, r_vdim=3, state=5, groups=1, conv=1, norm_groups=1, mlp=None),
              O.parallel_layer(heads=4, kv_heads=4, dim=4, vdim=9, chunk=1, rot_dims=0, r_heads=4, r_vdim=6, state=3, groups=4, conv=2, norm_groups=4, mlp=O.routed_mlp(4, 1, 6, count=2, keep=2)),
              O.parallel_layer(heads=6, kv_heads=3, dim=12, vdim=5, chunk=33, rot_dims=8, rot_base=3.0, r_heads=2, r_vdim=20, state=9, groups=2, conv=5, norm_groups=5, left_scale=-0.5, right_scale=0.25,
                               mlp=O.routed_mlp(9, 9, 5, count=1, keep=1, shared=11)),
              O.parallel_layer(mlp=O.dense_mlp(7))],
    "wide_heads": [O.parallel_layer(heads=8, kv_heads=2, dim=40, vdim=36, chunk=24, rot_dims=20, r_heads=4, r_vdim=40, state=36, groups=2, conv=4, norm_groups=2, mlp=O.routed_mlp(12, 3, 16, count=2, keep=1, shared=24)),
                   O.parallel_layer(heads=2, kv_heads=1, dim=70, vdim=3, chunk=10, rot_dims=70, r_heads=2, r_vdim=66, state=20, groups=1, conv=3, norm_groups=1, mlp=O.dense_mlp(50))],
}


@pytest.mark.gpu
@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("exact", [True, False])
def test_prompt_portions_and_decoding_agree_with_the_oracle(tmp_path, variant, exact):
    """the same 90 tokens as one prompt (cut by the pass width of 32), in portions of changing size (down to two tokens, inside and across chunks), and one by one"""
    m = small_model(seed=11, layers=VARIANTS[variant], width=64 if variant == "wide_heads" else 40)
    rng = np.random.default_rng(2)
    toks = [int(t) for t in rng.integers(0, 89, 90)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=128, n_batch=32, exact=exact)
    whole = e.ctx.feed(toks, 0, 0)
    assert within(logit_err(whole, want), exact)
    e.ctx.seq_rm(0, -1, -1)
    parts, a = [], 0
    for n in [2, 17, 3, 16, 31, 2, 5] * 3:
        if a >= 70:
            break
        parts.append(e.ctx.feed(toks[a:a + n], a, 0))
        a += n
    parts += [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(a, 90)]
    cut = np.concatenate(parts)
    assert within(logit_err(cut, want), exact)
    assert within(logit_err(cut, whole.astype(np.float64)), exact, 2e-5 if exact else 2e-2)     # the cut itself changes nothing beyond rounding
    e.ctx.seq_rm(0, -1, -1)
    single = np.concatenate([e.ctx.feed(toks[i:i + 1], i, 0) for i in range(40)])               # the first tokens of a sequence, one by one
    assert within(logit_err(single, want[:40]), exact)
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_a_wider_model_with_long_passes(tmp_path, exact):
    """sizes that reach the kernels' other paths: passes of 160 tokens (staged matrix-core products, grouped experts, the recurrence cut into pieces, the two-kernel convolution),
    two tiles of visible keys per chunk, several value columns per thread; then portions and single tokens across the chunk borders at 48, 96, ... and 100, 200"""
    layers = [O.parallel_layer(heads=6, kv_heads=3, dim=48, vdim=40, chunk=48, rot_dims=24, rot_base=500.0, scale=0.2, r_heads=6, r_vdim=32, state=40, groups=3, conv=4, norm_groups=2,
                               mlp=O.routed_mlp(12, 3, 40, count=3, keep=2, shared=56)),
              O.parallel_layer(heads=4, kv_heads=1, dim=72, vdim=80, chunk=100, rot_dims=72, rot_base=9000.0, scale=0.15, r_heads=8, r_vdim=24, state=72, groups=2, conv=3, norm_groups=4, mlp=O.dense_mlp(208)),
              O.parallel_layer(heads=6, kv_heads=3, dim=48, vdim=40, chunk=48, rot_dims=24, rot_base=500.0, scale=0.2, r_heads=6, r_vdim=32, state=40, groups=3, conv=4, norm_groups=2,
                               mlp=O.routed_mlp(12, 3, 40, count=3, keep=2, shared=56))]
    m = small_model(seed=91, layers=layers, width=192, vocab=301)
    rng = np.random.default_rng(17)
    toks = [int(t) for t in rng.integers(0, 301, 260)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=288, n_batch=160, exact=exact)
    whole = e.ctx.feed(toks, 0, 0)
    assert within(logit_err(whole, want), exact)
    e.ctx.seq_rm(0, -1, -1)
    cut = np.concatenate([e.ctx.feed(toks[:91], 0, 0), e.ctx.feed(toks[91:97], 91, 0), e.ctx.feed(toks[97:198], 97, 0)] + [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(198, 260)])
    assert within(logit_err(cut, want), exact)
    assert within(logit_err(cut, whole.astype(np.float64)), exact, 2e-5 if exact else 2e-2)
    e.close()


@pytest.mark.gpu
def test_residual_stream_layer_by_layer(tmp_path):
    """models cut after 1, 2, ... layers give the oracle's logits, so the first wrong layer would be named (each cut model keeps its own depth-average factors)"""
    full = small_model(seed=4)
    toks = [5, 17, 3, 88, 0, 41, 41, 7, 9, 9, 30]
    for n in range(1, 5):
        m = {"config": dict(full["config"], layers=full["config"]["layers"][:n]), "tensors": full["tensors"]}
        e = Engine(tmp_path, m, n_ctx=32, n_batch=8, name="cut%d" % n)
        assert logit_err(e.ctx.feed(toks, 0, 0), O.run(m, toks)).max() < TOL[True], n
        e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_batches_of_unequal_requests_equal_each_alone(tmp_path, exact):
    m = small_model(seed=21)
    rng = np.random.default_rng(8)
    reqs = [[int(t) for t in rng.integers(0, 89, n)] for n in (23, 5, 14)]
    want = [O.run(m, r) for r in reqs]
    e = Engine(tmp_path, m, n_ctx=128, n_batch=64, exact=exact)
    first = [9, 2, 14]
    toks = sum((r[:n] for r, n in zip(reqs, first)), [])
    pos = sum((list(range(n)) for n in first), [])
    seqs = sum(([[s]] * n for s, n in enumerate(first)), [])
    lg = e.ctx.decode(toks, pos, seqs)
    at = 0
    errs = []
    for s, n in enumerate(first):
        errs.append(logit_err(lg[at:at + n], want[s][:n]))
        at += n
    extra = [int(t) for t in rng.integers(0, 89, 6)]
    toks = reqs[1][2:] + extra + reqs[0][9:]
    pos = list(range(2, 5)) + list(range(6)) + list(range(9, 23))
    seqs = [[1]] * 3 + [[3]] * 6 + [[0]] * 14
    lg = e.ctx.decode(toks, pos, seqs)
    errs += [logit_err(lg[:3], want[1][2:]), logit_err(lg[3:9], O.run(m, extra)), logit_err(lg[9:], want[0][9:])]
    assert within(np.concatenate(errs), exact), [float(x.max()) for x in errs]
    e.close()


@pytest.mark.gpu
def test_freed_cells_and_slots_are_used_again(tmp_path):
    """more requests than slots and cells, one after the other and interleaved: a finished request gives back what it held, the next one starts from nothing (no key, no
    convolution input, no state of the earlier owner)"""
    m = small_model(seed=31)
    rng = np.random.default_rng(9)
    e = Engine(tmp_path, m, n_ctx=48, n_batch=16, slots=2)
    for round_ in range(5):
        a = [int(t) for t in rng.integers(0, 89, 20 + round_)]
        b = [int(t) for t in rng.integers(0, 89, 11)]
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
    a = [int(t) for t in rng.integers(0, 89, 12)]
    e.ctx.feed(a[:8], 0, 0)
    e.ctx.seq_cp(0, 1, -1, -1)                                      # a copy of a sequence (cells shared, state and convolution inputs copied) continues like the original
    assert logit_err(e.ctx.feed(a[8:] + [50, 51], 8, 1), O.run(m, a + [50, 51])[8:]).max() < TOL[True]
    assert logit_err(e.ctx.feed(a[8:] + [60], 8, 0), O.run(m, a + [60])[8:]).max() < TOL[True]
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_chunk_borders_show_in_prompts_and_in_decoding(tmp_path, exact):
    """sharp weights (a large score scale, a head bias that silences most keys) over several hundred tokens, chunk sizes that are no divisors of the pass width: a key that is
    wrongly seen or lost at a chunk's border, or a state that forgets, shows far above rounding — the same model with chunks one position longer is far away"""
    layers = [O.parallel_layer(heads=2, kv_heads=1, dim=8, vdim=8, chunk=50, rot_dims=4, scale=3.0, r_heads=2, r_vdim=4, state=4, groups=1, conv=4, mlp=None),
              O.parallel_layer(heads=3, kv_heads=3, dim=4, vdim=6, chunk=37, rot_dims=2, scale=4.0, mlp=ROUTED)]
    m = small_model(seed=41, layers=layers, width=32)
    for i in range(2):
        m["tensors"]["l%d.mix.left.pb" % i] = O.bf16_round((m["tensors"]["l%d.mix.left.pb" % i] - 2.0).astype(np.float32)).astype(np.float64)
    rng = np.random.default_rng(12)
    toks = [int(t) for t in rng.integers(0, 89, 330)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=340, n_batch=128, exact=exact)
    got = np.concatenate([e.ctx.feed(toks[:290], 0, 0)] + [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(290, 330)])       # decoding passes positions 296 and 300: a border of each layer
    err = logit_err(got, want)
    assert err.max() < TOL[exact] if exact else (np.quantile(err, 0.97) < TOL[exact] and err.max() < 10 * TOL[exact])
    longer = json.loads(json.dumps(m["config"]))
    longer["layers"][0]["mixer"]["left"]["mask"]["size"] = 51
    off = logit_err(got, O.run({"config": longer, "tensors": m["tensors"]}, toks))
    assert off[[50, 100, 299, 300]].min() > (100 if exact else 2) * TOL[exact]                    # (a chunk that is one position off would be seen, in the prompt and among the decoded tokens)
    e.close()


@pytest.mark.gpu
def test_long_decoding_token_by_token(tmp_path):
    m = small_model(seed=45)
    rng = np.random.default_rng(13)
    toks = [int(t) for t in rng.integers(0, 89, 200)]
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
    toks = [int(t) for t in rng.integers(0, 89, 60)]
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
    m = small_model(seed=81, layers=VARIANTS["edges"])
    folder, out = str(tmp_path / "model"), str(tmp_path / "out")
    write(folder, m)
    rng = np.random.default_rng(5)
    a, b = [int(t) for t in rng.integers(0, 89, 41)], [int(t) for t in rng.integers(0, 89, 9)]
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
        got = np.fromfile(os.path.join(out, "%d.f32" % k), "<f4").reshape(-1, 89)
        assert got.shape == w.shape and np.median(logit_err(got, w)) < TOL[dtype == "float32"] and (dtype != "float32" or logit_err(got, w).max() < TOL[True]), k
