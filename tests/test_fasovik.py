"""The Fasovik design (hybrid of latent attention and lightning layers with routed experts) on the engine, held to the plain numpy restatement in
tests/fasovik_oracle.py: every mechanism alone through its operator, then whole models through llama_decode — prompts against token-by-token
decoding, portions down to two tokens, batches of unequal requests, cells and state slots that are freed and used again, long decoding, greedy
generation.  Models are small, random and made here; sizes are chosen so that nothing that could be mixed up is equal (heads, dim, vdim, ranks)."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from pipeinfer_amd import lib as L, llama as LL
from tests import fasovik_oracle as O

BF16 = 30


# ---- helpers ------------------------------------------------------------------------------------------------------------------
def bf(rng, *shape, s=1.0):
    return O.bf16_round((rng.standard_normal(shape) * s).astype(np.float32))


def rel_rms(got, want):
    d = np.asarray(got, np.float64) - np.asarray(want, np.float64)
    return float(np.sqrt((d * d).mean()) / (np.sqrt((np.asarray(want, np.float64) ** 2).mean()) + 1e-30))


def logit_err(got, want):
    """per row: rms of the difference with its mean taken off (a constant shift of a row of logits changes nothing), relative to the rows' spread"""
    d = np.asarray(got, np.float64) - want
    d = d - d.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / (want - want.mean(-1, keepdims=True)).std()


TOL = {True: 3e-4, False: 4e-2}          # exact (fp32) / serving precision (bfloat16 matrix inputs)


def layer(kind, heads, dim, vdim, rank=None, scale=None, decay=None, mlp=None, weights_of=None):
    mix = {"heads": heads, "dim": dim, "vdim": vdim}
    if kind == "latent_attention":
        mix.update(kv_rank=rank, scale=scale if scale is not None else 1.0 / np.sqrt(dim))
    else:
        mix["decay"] = list(decay if decay is not None else np.linspace(0.7, 0.995, heads))
    d = {"type": kind, "mixer": mix, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


MOE = {"ff": 24, "experts": 5, "identity": 2, "top": 3}


def small_model(seed=0, width=48, vocab=97, layers=None, **kw):
    rng = np.random.default_rng(seed)
    layers = layers or [layer("latent_attention", 3, 8, 10, rank=20, mlp=MOE),
                        layer("lightning", 2, 12, 6, mlp=MOE),
                        layer("latent_attention", 3, 8, 10, rank=20, mlp=None),
                        layer("lightning", 2, 12, 6, mlp=MOE, weights_of=1)]
    return O.random_model(rng, vocab, width, layers, **kw)


class Engine:
    def __init__(self, tmp_path, model, n_ctx=256, n_batch=64, exact=True, slots=4, name="m"):
        folder = os.path.join(str(tmp_path), name)
        O.write_model(folder, model["config"], {k: v.astype(np.float32) if v.dtype.kind == "f" else v for k, v in model["tensors"].items()})
        self.model = LL.Model(folder)
        self.ctx = LL.Context(self.model, n_ctx=n_ctx, n_batch=n_batch)
        self.ctx.set_state_slots(slots)
        self.ctx.set_precision(exact)

    def close(self):
        self.ctx.free()
        self.model.free()


# ---- without a GPU: the description reader and the slot table ---------------------------------------------------------------------
def test_model_folder_is_read_and_described(tmp_path):
    m = small_model()
    folder = str(tmp_path / "m")
    O.write_model(folder, m["config"], {k: v.astype(np.float32) for k, v in m["tensors"].items()})
    for path in (folder, os.path.join(folder, "config.json")):
        mod = LL.Model(path)
        assert mod.n_vocab == 97
        buf = C.create_string_buffer(64)
        mod.lib.llama_model_desc.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        mod.lib.llama_model_desc(mod.h, buf, 64)
        assert buf.value.startswith(b"fasovik")
        mod.free()
    back = O.read_model(folder)
    assert all(np.array_equal(back["tensors"][k], m["tensors"][k]) for k in m["tensors"])


@pytest.mark.parametrize("breakage", ["mixer", "top", "decay", "weights_of", "arch", "kind"])
def test_a_wrong_description_is_refused(tmp_path, breakage):
    m = small_model()
    cfg = json.loads(json.dumps(m["config"]))
    if breakage == "mixer":
        cfg["layers"][0]["type"] = "sliding"
    elif breakage == "top":
        cfg["layers"][0]["mlp"]["router"]["top"] = 99
    elif breakage == "decay":
        cfg["layers"][1]["mixer"]["decay"] = [0.5]
    elif breakage == "weights_of":
        cfg["layers"][3]["weights_of"] = 0            # a latent-attention layer's tensors for a lightning layer
    elif breakage == "arch":
        cfg["architecture"] = "Other"
    elif breakage == "kind":
        cfg["layers"][0]["mlp"]["kind"] = "dense"
    folder = str(tmp_path / "bad")
    O.write_model(folder, cfg, {k: v.astype(np.float32) for k, v in m["tensors"].items()})
    with pytest.raises(L.PipeInferError):
        LL.Model(folder)


def test_state_slots_are_handed_out_freed_and_reused():
    lib = LL.api()
    lib.pi_stateslots_new.restype = C.c_void_p
    for n in ("free", "acquire", "take_fresh", "find", "used", "release", "keep", "clear"):
        getattr(lib, "pi_stateslots_" + n).argtypes = [C.c_void_p] + [C.c_int] * (0 if n in ("free", "used", "clear") else 1)
    s = lib.pi_stateslots_new(3)
    a, b = lib.pi_stateslots_acquire(s, 7), lib.pi_stateslots_acquire(s, 9)
    assert (a, b) == (0, 1) and lib.pi_stateslots_acquire(s, 7) == 0
    assert lib.pi_stateslots_take_fresh(s, a) == 1 and lib.pi_stateslots_take_fresh(s, a) == 0          # told once
    c = lib.pi_stateslots_acquire(s, 11)
    assert c == 2 and lib.pi_stateslots_acquire(s, 12) == -1 and lib.pi_stateslots_used(s) == 3
    lib.pi_stateslots_release(s, 9)
    assert lib.pi_stateslots_find(s, 9) == -1 and lib.pi_stateslots_used(s) == 2
    d = lib.pi_stateslots_acquire(s, 12)
    assert d == 1 and lib.pi_stateslots_take_fresh(s, d) == 1                                           # the freed slot again, from zero
    lib.pi_stateslots_keep(s, 12)
    assert lib.pi_stateslots_used(s) == 1 and lib.pi_stateslots_find(s, 12) == 1 and lib.pi_stateslots_find(s, 7) == -1
    lib.pi_stateslots_clear(s)
    assert lib.pi_stateslots_used(s) == 0
    lib.pi_stateslots_free(s)


def test_oracle_mechanisms_behave_as_stated():
    """the restatement itself: an identity expert returns its input, a very negative sink leaves a plain soft-max, the decay of 1 sums outer products"""
    rng = np.random.default_rng(3)
    m = small_model(seed=3)
    T, cfg = m["tensors"], m["config"]
    h = rng.standard_normal(48)
    T["l0.mlp.correction"] = np.array([-9.0] * 5 + [9.0, 8.0])         # the correction decides the choice, not the weight
    idx, w = O.moe_route(T, "l0.", dict(cfg["layers"][0]["mlp"], router={"experts": 5, "identity": 2, "top": 2}), h)
    assert idx == [5, 6] and np.allclose(w, O.softmax(T["l0.mlp.router"] @ h)[[5, 6]])
    out = O.moe(T, "l0.", dict(cfg["layers"][0]["mlp"], router={"experts": 5, "identity": 2, "top": 2}), h)
    assert np.allclose(out, sum(w) * h)
    mix = dict(cfg["layers"][1]["mixer"], decay=[1.0, 1.0])
    st = np.zeros((2, 12, 6))
    O.lightning_step(T, "l1.", mix, 1e-5, h, st)
    first = st.copy()
    O.lightning_step(T, "l1.", mix, 1e-5, h, st)
    assert np.allclose(st, 2 * first)


# ---- operators alone ------------------------------------------------------------------------------------------------------------------
def gpu():
    from tests import gpu_util as U
    return U, U.init()


def upload_bf16(lib, w):
    u = (np.ascontiguousarray(w, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    h = lib.pi_weight_upload(BF16, w.shape[1], w.shape[0], u.ctypes.data_as(C.c_void_p), None)
    assert h, lib.pi_last_error()
    return h


@pytest.mark.gpu
@pytest.mark.parametrize("K,N,T", [(40, 37, 1), (33, 10, 3), (512, 70, 5), (1024, 130, 8), (96, 200, 17), (64, 64, 64), (520, 33, 150), (256, 300, 200), (72, 130, 129)])
@pytest.mark.parametrize("exact", [True, False])
def test_dense_every_kernel_and_width(K, N, T, exact):
    U, lib = gpu()
    rng = np.random.default_rng(K + N + T)
    w, x = bf(rng, N, K, s=0.2), rng.standard_normal((T, K + 3)).astype(np.float32)          # (rows of x three floats apart from dense)
    wd, xd, od = upload_bf16(lib, w), U.Dev(x), U.Dev(nbytes=4 * T * (N + 5))
    for act_a, rows_a, act_b in ((0, N, 0), (1, N // 2, 2), (3, N, 0)):
        L.check(lib.pi_op_dense(wd, xd.ptr, K + 3, T, od.ptr, N + 5, act_a, rows_a, act_b, int(exact), None))
        got = od.get(np.float32, (T, N + 5))[:, :N]
        xin = x[:, :K].astype(np.float64) if exact else O.bf16_round(x[:, :K]).astype(np.float64)
        z = xin @ w.astype(np.float64).T
        f = {0: lambda v: v, 1: O.silu, 2: O.sigmoid, 3: lambda v: np.maximum(v, 0) ** 2}
        want = np.concatenate([f[act_a](z[:, :rows_a]), f[act_b](z[:, rows_a:])], axis=1)
        assert rel_rms(got, want) < 2e-6, (act_a, rel_rms(got, want))
    lib.pi_weight_free(wd)


@pytest.mark.gpu
def test_embedding_rows_are_scaled():
    U, lib = gpu()
    rng = np.random.default_rng(1)
    w = bf(rng, 50, 24)
    toks = np.array([3, 49, 0, 3], np.int32)
    wd, td, od = upload_bf16(lib, w), U.Dev(toks), U.Dev(nbytes=4 * 4 * 24)
    L.check(lib.pi_op_embed(wd, td.ptr, 4, 2.5, od.ptr, None))
    assert np.array_equal(od.get(np.float32, (4, 24)), w[toks] * np.float32(2.5))
    lib.pi_weight_free(wd)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [7, 96, 300, 1000])
def test_rms_scale_offsets_gate_and_residual(n):
    U, lib = gpu()
    rng = np.random.default_rng(n)
    T = 5
    x, w, g, r = (rng.standard_normal(s).astype(np.float32) for s in ((T, n + 2), (n,), (T, n), (T, n)))
    xd, wd, gd, rd, od = U.Dev(x), U.Dev(w), U.Dev(g), U.Dev(r), U.Dev(nbytes=4 * T * n)
    norm = x[:, :n].astype(np.float64) / np.sqrt((x[:, :n].astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-3)
    L.check(lib.pi_op_rms_scale(xd.ptr, n + 2, wd.ptr, 1.0, 1e-3, n, T, None, 0, rd.ptr, n, 0.3, od.ptr, n, None, 0, None))
    assert rel_rms(od.get(np.float32, (T, n)), r + 0.3 * norm * (1.0 + w)) < 1e-6
    L.check(lib.pi_op_rms_scale(xd.ptr, n + 2, wd.ptr, 0.0, 1e-3, n, T, gd.ptr, n, None, 0, 1.0, od.ptr, n, None, 0, None))
    assert rel_rms(od.get(np.float32, (T, n)), norm * w * g) < 1e-6
    # rows written into cache cells: cell table {first cell, n_kv, n_tok, 0}
    dyn, cache = U.Dev(np.array([6, 11, T, 0], np.int32)), U.Dev(nbytes=4 * 16 * n)
    L.check(lib.pi_op_rms_scale(xd.ptr, n + 2, wd.ptr, 0.0, 1e-3, n, T, None, 0, None, 0, 1.0, cache.ptr, n, dyn.ptr, 1, None))
    c = cache.get(np.float32, (16, n))
    assert rel_rms(c[6:11], norm * w) < 1e-6 and not c[:6].any() and not c[11:].any()


def lightning_ref(q, k, v, decay, state):
    out = np.zeros((q.shape[0], q.shape[1], v.shape[2]))
    for t in range(q.shape[0]):
        for h in range(q.shape[1]):
            state[h] = decay[h] * state[h] + np.outer(k[t, h], v[t, h])
            out[t, h] = state[h].T @ q[t, h]
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("H,D,V", [(1, 5, 3), (2, 16, 70), (3, 24, 32), (2, 48, 10), (2, 100, 33), (1, 200, 130)])
def test_linear_attention_states_segments_and_slots(H, D, V):
    U, lib = gpu()
    rng = np.random.default_rng(H * D + V)
    slots, stride = 5, 2 * H * D + H * V + 4
    decay = np.linspace(0.5, 0.999, H).astype(np.float32)
    state = rng.standard_normal((slots, H, D, V)).astype(np.float32)                    # whatever an earlier owner of the slots left behind
    sd, dd = U.Dev(state), U.Dev(decay)
    ref = {s: None for s in range(slots)}

    def run(rec):
        T = len(rec)
        buf = (rng.standard_normal((T, stride)) * 0.5).astype(np.float32)
        q, k, v = (buf[:, a:b].reshape(T, H, -1) for a, b in ((0, H * D), (H * D, 2 * H * D), (2 * H * D, 2 * H * D + H * V)))
        bd, rdv, od = U.Dev(buf), U.Dev(np.array(rec, np.int32)), U.Dev(nbytes=4 * T * H * V)
        base = bd.ptr
        nscr = lib.pi_op_linear_attention_scratch_floats(H, D, V, T, slots)
        scr = U.Dev(nbytes=4 * nscr)
        L.check(lib.pi_op_linear_attention(base, base + 4 * H * D, base + 8 * H * D, stride, H, D, V, dd.ptr, sd.ptr, rdv.ptr, T, slots, scr.ptr, nscr, od.ptr, H * V, None))
        got = od.get(np.float32, (T, H, V))
        t = 0
        while t < T:
            s = rec[t] & ~(1 << 30)
            e = t
            while e < T and (rec[e] & ~(1 << 30)) == s:
                e += 1
            if rec[t] & (1 << 30):
                ref[s] = np.zeros((H, D, V))
            want = lightning_ref(q[t:e].astype(np.float64), k[t:e].astype(np.float64), v[t:e].astype(np.float64), decay.astype(np.float64), ref[s])
            assert rel_rms(got[t:e], want) < 2e-5, (s, t, e)
            t = e
    F = 1 << 30
    run([2 | F] + [2] * 20 + [4 | F] + [4] * 2 + [0 | F])             # three sequences of unequal length in one pass, fresh slots over garbage
    run([0] * 70 + [3 | F] + [3] * 32 + [4] * 33)                   # a long pass: runs cut into pieces of 32 (2 full + 6 | exactly 33 = 32 + 1 | 32 + 1), carried and fresh
    run([4] * 17)                                                   # one of them goes on: a tile of 16 and one more
    run([0] + [2] * 3 + [4])                                        # single tokens of each
    run([2 | F] + [2] * 40)                                         # slot 2 handed to a new sequence: from zero again
    assert rel_rms(sd.get(np.float32, (slots, H, D, V))[2], ref[2]) < 2e-5
    assert np.array_equal(sd.get(np.float32, (slots, H, D, V))[1], state[1])               # a slot nobody named is untouched


def latent_ref(q, cache, vis, wuk, wuv, sink, scale, H, D, V):
    T = q.shape[0]
    out = np.zeros((T, H, V))
    for t in range(T):
        cells = np.nonzero(vis[t])[0]
        c = cache[cells].astype(np.float64)
        for h in range(H):
            kk, vv = c @ wuk[h * D:(h + 1) * D].T, c @ wuv[h * V:(h + 1) * V].T
            s = kk @ q[t, h * D:(h + 1) * D] * scale
            m = max(s.max(), sink[h]) if len(s) else sink[h]
            e = np.exp(s - m)
            out[t, h] = (e / (e.sum() + np.exp(sink[h] - m))) @ vv if len(s) else 0
    return out.reshape(T, H * V)


def pack_mask(vis, n_kv):
    words = (n_kv + 31) // 32
    m = np.zeros((vis.shape[0], words), np.uint32)
    for t, j in zip(*np.nonzero(vis)):
        m[t, j >> 5] |= np.uint32(1 << (j & 31))
    return m


@pytest.mark.gpu
@pytest.mark.parametrize("H,D,V,R,T,n_kv", [(1, 4, 6, 10, 1, 33), (3, 8, 10, 20, 5, 70), (9, 16, 12, 96, 9, 300), (6, 32, 24, 64, 20, 700), (2, 24, 40, 130, 3, 1500), (16, 8, 8, 300, 12, 2500),
                                            (5, 8, 8, 520, 2, 200), (17, 4, 4, 32, 33, 90), (3, 8, 8, 48, 2, 4500)])
def test_latent_attention_against_explicit_keys_and_values(H, D, V, R, T, n_kv):
    U, lib = gpu()
    rng = np.random.default_rng(R + T)
    n_ctx = n_kv + 37                                             # cells behind n_kv hold garbage that must never be read
    cache = rng.standard_normal((n_ctx, R)).astype(np.float32)
    cache[n_kv:] = np.nan
    wuk, wuv = bf(rng, H * D, R, s=0.3), bf(rng, H * V, R, s=0.3)
    q = rng.standard_normal((T, H * D + 7)).astype(np.float32)
    sink = rng.standard_normal(H).astype(np.float32)
    vis = rng.random((T, n_ctx)) < 0.6
    vis[:, n_kv:] = False
    vis[0, :] = False
    vis[0, n_kv - 1] = True                                       # one token sees a single, last cell
    if T > 1:
        vis[1, :n_kv] = True
    for exactly_far in (False, True):
        if exactly_far:                                           # one far cell must win against hundreds: its latent is the query's own direction, scaled up
            qa = q[-1, :D].astype(np.float64) @ wuk[:D].astype(np.float64)
            cache[3] = (qa / np.linalg.norm(qa) * 30).astype(np.float32)
            vis[-1, 3] = True
        dyn = np.array([0, n_kv, T, 0], np.int32)
        args = [U.Dev(a) for a in (q, cache, pack_mask(vis, n_ctx), sink, dyn)]
        ukd, uvd, od = upload_bf16(lib, wuk), upload_bf16(lib, wuv), U.Dev(nbytes=4 * T * H * V)
        nscr = lib.pi_op_latent_attention_scratch_floats(H, R, T, n_ctx)
        scr = U.Dev(nbytes=4 * nscr)
        L.check(lib.pi_op_latent_attention(args[0].ptr, H * D + 7, args[1].ptr, args[2].ptr, ukd, uvd, args[3].ptr, 0.37, H, D, V, R, T, n_ctx, scr.ptr, nscr, od.ptr, H * V, args[4].ptr, None))
        got = od.get(np.float32, (T, H * V))
        want = latent_ref(q[:, :H * D].astype(np.float64), np.nan_to_num(cache), vis, wuk.astype(np.float64), wuv.astype(np.float64), sink.astype(np.float64), 0.37, H, D, V)
        assert np.isfinite(got).all() and rel_rms(got, want) < 5e-5, rel_rms(got, want)
        if exactly_far:
            without = vis.copy()
            without[-1, 3] = False
            other = latent_ref(q[:, :H * D].astype(np.float64), np.nan_to_num(cache), without, wuk.astype(np.float64), wuv.astype(np.float64), sink.astype(np.float64), 0.37, H, D, V)
            assert rel_rms(other[-1], want[-1]) > 0.1                 # (the test would notice that cell going missing)
        lib.pi_weight_free(ukd); lib.pi_weight_free(uvd)


@pytest.mark.gpu
def test_latent_attention_sink_takes_its_share():
    """a large sink swallows most of the probability mass (outputs shrink towards zero), a very negative one leaves the plain soft-max"""
    U, lib = gpu()
    rng = np.random.default_rng(5)
    H, D, V, R, n = 2, 8, 8, 16, 40
    cache, q = rng.standard_normal((n, R)).astype(np.float32), rng.standard_normal((1, H * D)).astype(np.float32)
    wuk, wuv = bf(rng, H * D, R, s=0.3), bf(rng, H * V, R, s=0.3)
    vis = np.ones((1, n), bool)
    outs = []
    for sk in (-60.0, 0.0, 12.0):
        sink = np.full(H, sk, np.float32)
        ukd, uvd, od = upload_bf16(lib, wuk), upload_bf16(lib, wuv), U.Dev(nbytes=4 * H * V)
        a = [U.Dev(x) for x in (q, cache, pack_mask(vis, n), sink, np.array([0, n, 1, 0], np.int32))]
        nscr = lib.pi_op_latent_attention_scratch_floats(H, R, 1, n)
        scr = U.Dev(nbytes=4 * nscr)
        L.check(lib.pi_op_latent_attention(a[0].ptr, H * D, a[1].ptr, a[2].ptr, ukd, uvd, a[3].ptr, 0.5, H, D, V, R, 1, n, scr.ptr, nscr, od.ptr, H * V, a[4].ptr, None))
        outs.append(od.get(np.float32, (1, H * V)))
        want = latent_ref(q.astype(np.float64), cache, vis, wuk.astype(np.float64), wuv.astype(np.float64), sink.astype(np.float64), 0.5, H, D, V)
        assert rel_rms(outs[-1], want) < 5e-5
    assert np.abs(outs[2]).max() < 0.05 * np.abs(outs[0]).max() and rel_rms(outs[1], outs[0]) > 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("E,I,top,ff,width", [(5, 2, 3, 24, 48), (1, 0, 1, 7, 33), (4, 4, 2, 64, 96), (0, 3, 2, 0, 40), (70, 3, 6, 16, 64)])
@pytest.mark.parametrize("exact", [True, False])
def test_router_and_experts(E, I, top, ff, width, exact):
    U, lib = gpu()
    rng = np.random.default_rng(E * 7 + I)
    T, n_out = 6, E + I
    x = rng.standard_normal((T, width)).astype(np.float32)
    router, corr = bf(rng, n_out, width, s=0.4), bf(rng, n_out, s=0.3)
    ups, downs = bf(rng, max(E, 1) * max(ff, 1), width, s=0.2), bf(rng, max(E, 1) * width, max(ff, 1), s=0.2)
    tens = {"l0.mlp.router": router.astype(np.float64), "l0.mlp.correction": corr.astype(np.float64)}
    for e in range(E):
        tens["l0.mlp.e%d.up" % e] = ups[e * ff:(e + 1) * ff].astype(np.float64)
        tens["l0.mlp.e%d.down" % e] = downs[e * width:(e + 1) * width].astype(np.float64)
    mlp = {"router": {"experts": E, "identity": I, "top": top}}
    rd, cd, xd = upload_bf16(lib, router), U.Dev(corr), U.Dev(x)
    sel, selw = U.Dev(nbytes=4 * T * top), U.Dev(nbytes=4 * T * top)
    L.check(lib.pi_op_moe_route(rd, cd.ptr, xd.ptr, width, T, top, int(exact), sel.ptr, selw.ptr, None))
    gs, gw = sel.get(np.int32, (T, top)), selw.get(np.float32, (T, top))
    xin = x.astype(np.float64) if exact else O.bf16_round(x).astype(np.float64)
    for t in range(T):
        idx, w = O.moe_route(tens, "l0.", mlp, xin[t])
        assert list(gs[t]) == idx and np.allclose(gw[t], w, rtol=2e-5)
    ud = upload_bf16(lib, ups) if E else None
    dd = upload_bf16(lib, downs) if E else None
    upb, od = U.Dev(nbytes=4 * T * top * max(ff, 1)), U.Dev(nbytes=4 * T * width)
    L.check(lib.pi_op_moe_experts(ud, dd, E, ff, xd.ptr, width, sel.ptr, selw.ptr, T, top, int(exact), upb.ptr, od.ptr, width, None))
    got = od.get(np.float32, (T, width))
    want = np.zeros((T, width))
    for t in range(T):
        for e, w in zip(gs[t], gw[t].astype(np.float64)):
            if e >= E:
                want[t] += w * x[t]
            else:
                u = np.maximum(tens["l0.mlp.e%d.up" % e] @ xin[t], 0) ** 2
                want[t] += w * (tens["l0.mlp.e%d.down" % e] @ (u if exact else O.bf16_round(u.astype(np.float32)).astype(np.float64)))
    assert rel_rms(got, want) < (1e-5 if exact else 2e-3)


# ---- whole models through llama_decode ------------------------------------------------------------------------------------------------------
VARIANTS = {
    "mixed": None,
    "other_sizes": [layer("lightning", 1, 20, 7, decay=[0.93], mlp={"ff": 9, "experts": 2, "identity": 0, "top": 1}),
                    layer("latent_attention", 1, 6, 5, rank=9, scale=0.9, mlp={"ff": 16, "experts": 3, "identity": 3, "top": 4}),
                    layer("latent_attention", 5, 4, 12, rank=33, scale=0.25, mlp=None),
                    layer("lightning", 4, 5, 17, mlp=None),
                    layer("latent_attention", 1, 6, 5, rank=9, scale=0.9, mlp={"ff": 16, "experts": 3, "identity": 3, "top": 4}, weights_of=1)],
    "only_lightning": [layer("lightning", 3, 6, 9, mlp=None), layer("lightning", 3, 6, 9, mlp=MOE, weights_of=2), layer("lightning", 3, 6, 9, mlp=MOE)],      # (tensors of a LATER layer)
    "only_latent": [layer("latent_attention", 5, 6, 4, rank=14, mlp=None), layer("latent_attention", 2, 10, 12, rank=24, scale=0.5, mlp=MOE),
                    layer("latent_attention", 2, 10, 12, rank=24, scale=0.5, mlp=MOE, weights_of=1), layer("latent_attention", 2, 10, 12, rank=24, scale=0.5, mlp=MOE, weights_of=2)],
    "only_identity": [layer("latent_attention", 2, 8, 8, rank=12, mlp={"ff": 0, "experts": 0, "identity": 3, "top": 2}),
                      layer("lightning", 2, 8, 8, mlp={"ff": 8, "experts": 4, "identity": 1, "top": 5})],
}


@pytest.mark.gpu
@pytest.mark.parametrize("variant", list(VARIANTS))
@pytest.mark.parametrize("exact", [True, False])
def test_prompt_portions_and_decoding_agree_with_the_oracle(tmp_path, variant, exact):
    """the same 90 tokens as one prompt, in portions of changing size (down to two tokens, across the 16-token tile of the recurrence and the pass width), and one by one"""
    m = small_model(seed=11, layers=VARIANTS[variant], width=40 if variant == "other_sizes" else 48)
    rng = np.random.default_rng(2)
    toks = [int(t) for t in rng.integers(0, 97, 90)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=128, n_batch=32, exact=exact)
    whole = e.ctx.feed(toks, 0, 0)
    assert logit_err(whole, want).max() < TOL[exact]
    e.ctx.seq_rm(0, -1, -1)
    parts, a = [], 0
    for n in [2, 17, 3, 16, 31, 2, 5] * 3:
        if a >= 70:
            break
        parts.append(e.ctx.feed(toks[a:a + n], a, 0))
        a += n
    parts += [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(a, 90)]
    cut = np.concatenate(parts)
    assert logit_err(cut, want).max() < TOL[exact]
    assert logit_err(cut, whole.astype(np.float64)).max() < (2e-5 if exact else 2e-2)          # the cut itself changes nothing beyond rounding
    e.ctx.seq_rm(0, -1, -1)
    single = np.concatenate([e.ctx.feed(toks[i:i + 1], i, 0) for i in range(40)])
    assert logit_err(single, want[:40]).max() < TOL[exact]
    e.close()


@pytest.mark.gpu
def test_residual_stream_layer_by_layer(tmp_path):
    """PI_TRACE-free check of the layers: models cut after 1, 2, ... layers give the oracle's logits, so the first wrong layer would be named"""
    full = small_model(seed=4)
    toks = [5, 17, 3, 96, 0, 41, 41, 7]
    for n in range(1, 4):                                           # (layer 3 borrows layer 1's tensors: covered by the full model elsewhere)
        m = {"config": dict(full["config"], layers=full["config"]["layers"][:n]), "tensors": full["tensors"]}
        e = Engine(tmp_path, m, n_ctx=32, n_batch=8, name="cut%d" % n)
        assert logit_err(e.ctx.feed(toks, 0, 0), O.run(m, toks)).max() < TOL[True], n
        e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_batches_of_unequal_requests_equal_each_alone(tmp_path, exact):
    m = small_model(seed=21)
    rng = np.random.default_rng(8)
    reqs = [[int(t) for t in rng.integers(0, 97, n)] for n in (23, 5, 14)]
    want = [O.run(m, r) for r in reqs]
    e = Engine(tmp_path, m, n_ctx=128, n_batch=64, exact=exact)
    # pass 1: the first 9 / 2 / 14 tokens of the three requests in ONE batch; pass 2: the rest of two of them, with a fourth sequence starting meanwhile
    first = [9, 2, 14]
    toks = sum((r[:n] for r, n in zip(reqs, first)), [])
    pos = sum((list(range(n)) for n in first), [])
    seqs = sum(([[s]] * n for s, n in enumerate(first)), [])
    lg = e.ctx.decode(toks, pos, seqs)
    at = 0
    for s, n in enumerate(first):
        assert logit_err(lg[at:at + n], want[s][:n]).max() < TOL[exact], s
        at += n
    extra = [int(t) for t in rng.integers(0, 97, 6)]
    toks = reqs[1][2:] + extra + reqs[0][9:]
    pos = list(range(2, 5)) + list(range(6)) + list(range(9, 23))
    seqs = [[1]] * 3 + [[3]] * 6 + [[0]] * 14
    lg = e.ctx.decode(toks, pos, seqs)
    assert logit_err(lg[:3], want[1][2:]).max() < TOL[exact]
    assert logit_err(lg[3:9], O.run(m, extra)).max() < TOL[exact]
    assert logit_err(lg[9:], want[0][9:]).max() < TOL[exact]
    # a sequence whose tokens are not next to each other is refused, and nothing is lost by the refusal
    with pytest.raises(L.PipeInferError):
        e.ctx.decode([1, 2, 3], [23, 5, 24], [[0], [1], [0]])
    nxt = e.ctx.decode([7], [23], [[0]])
    assert logit_err(nxt, O.run(m, reqs[0] + [7])[-1:]).max() < TOL[exact]
    e.close()


@pytest.mark.gpu
def test_freed_cells_and_slots_are_used_again(tmp_path):
    """more requests than slots and cells, one after the other and interleaved: a finished request gives back what it held, the next one starts from nothing"""
    m = small_model(seed=31)
    rng = np.random.default_rng(9)
    e = Engine(tmp_path, m, n_ctx=48, n_batch=16, slots=2)
    for round_ in range(5):
        a = [int(t) for t in rng.integers(0, 97, 20 + round_)]
        b = [int(t) for t in rng.integers(0, 97, 11)]
        la = e.ctx.feed(a[:7], 0, 0)
        lb = e.ctx.feed(b, 0, 1)
        la = np.concatenate([la, e.ctx.feed(a[7:], 7, 0)])
        assert e.ctx.state_slots_used() == 2
        with pytest.raises(L.PipeInferError):                      # a third live sequence finds no slot ...
            e.ctx.decode([1], [0], [[2]])
        e.ctx.seq_rm(1, -1, -1)
        lc = e.ctx.feed(b[:5], 0, 2)                               # ... until one is given back
        for got, toks in ((la, a), (lb, b), (lc, b[:5])):
            assert logit_err(got, O.run(m, toks)).max() < TOL[True], round_
        e.ctx.seq_rm(0, -1, -1)
        e.ctx.seq_rm(2, -1, -1)
        assert e.ctx.state_slots_used() == 0
    # a sequence cannot be cut in the middle (its state is not kept per position): refused, and the sequence goes on unharmed
    a = [int(t) for t in rng.integers(0, 97, 12)]
    e.ctx.feed(a[:8], 0, 0)
    e.ctx.seq_rm(0, 4, -1)
    assert logit_err(e.ctx.feed(a[8:], 8, 0), O.run(m, a)[8:]).max() < TOL[True]
    # a copy of a sequence continues like the original
    e.ctx.seq_cp(0, 1, -1, -1)
    assert logit_err(e.ctx.feed([50, 51], 12, 1), O.run(m, a + [50, 51])[12:]).max() < TOL[True]
    assert logit_err(e.ctx.feed([60], 12, 0), O.run(m, a + [60])[12:]).max() < TOL[True]
    e.close()


@pytest.mark.gpu
@pytest.mark.parametrize("exact", [True, False])
def test_far_keys_and_strong_sinks_show_in_the_logits(tmp_path, exact):
    """sharp attention (a large score scale) over a few hundred tokens: a lost key, a lost sink or a state that forgets shows far above rounding.  The prompt is longer than the
    pass width and ends in single tokens."""
    layers = [layer("latent_attention", 2, 8, 8, rank=16, scale=2.5, mlp=None),
              layer("lightning", 2, 8, 8, decay=[0.999, 0.9], mlp=MOE),
              layer("latent_attention", 3, 4, 6, rank=8, scale=3.0, mlp=MOE)]
    m = small_model(seed=41, layers=layers, width=32)
    m["tensors"]["l0.mix.sink"] = O.bf16_round(np.array([4.0, -3.0], np.float32)).astype(np.float64)
    rng = np.random.default_rng(12)
    toks = [int(t) for t in rng.integers(0, 97, 330)]
    want = O.run(m, toks)
    e = Engine(tmp_path, m, n_ctx=340, n_batch=128, exact=exact)
    got = np.concatenate([e.ctx.feed(toks[:300], 0, 0)] + [e.ctx.feed(toks[i:i + 1], i, 0) for i in range(300, 330)])
    err = logit_err(got, want)
    # (scores this sharp magnify bfloat16 rounding, and a router's close call may then fall the other way at a few places: at serving precision nearly all places must be
    # within the tolerance and none far off; in fp32 every place is)
    assert err.max() < TOL[exact] if exact else (np.quantile(err, 0.97) < TOL[exact] and err.max() < 10 * TOL[exact])
    nosink = {"config": m["config"], "tensors": dict(m["tensors"], **{"l0.mix.sink": np.array([-50.0, -50.0])})}
    assert logit_err(got, O.run(nosink, toks)).max() > 0.2                       # (a lost sink would be seen)
    e.close()


@pytest.mark.gpu
def test_greedy_generation_through_the_engine(tmp_path):
    m = small_model(seed=51)
    prompt = [3, 14, 15, 92, 65, 35]
    e = Engine(tmp_path, m, n_ctx=160, n_batch=16, exact=True)
    got = e.ctx.generate(prompt, 120)
    want = O.greedy(m, prompt, 120)
    # (an arg-max between two nearly equal logits may fall either way in fp32 against float64: compare up to the first such place, which must be a near tie)
    k = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), len(want))
    if k < len(want):
        lg = O.run(m, prompt + want[:k])[-1]
        assert abs(lg[got[k]] - lg[want[k]]) < 1e-3 * np.abs(lg).max()
    assert k >= 20
    e.close()


@pytest.mark.gpu
def test_graph_replays_equal_eager_launches(tmp_path):
    """every pass width is captured once and replayed: replays, with other passes in between, give what eager launches give"""
    m = small_model(seed=61)
    rng = np.random.default_rng(3)
    toks = [int(t) for t in rng.integers(0, 97, 60)]
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
def test_generate_command_line_greedy_and_sampled(tmp_path, capsys):
    """the generation command: greedy ids equal the engine's own generate(); with a temperature the llama.h samplers pick from the top-k of the same logits, reproducibly per seed"""
    from pipeinfer_amd.tools import generate as G
    m = small_model(seed=71)
    folder = str(tmp_path / "g")
    O.write_model(folder, m["config"], {k: v.astype(np.float32) for k, v in m["tensors"].items()})
    assert G.main(["--model", folder, "--prompt-ids", "5,6,7", "--n-predict", "12", "--float32"]) == 0
    greedy = [int(t) for t in capsys.readouterr().out.strip().split(",")]
    want = O.greedy(m, [5, 6, 7], 12)
    k = next((i for i, (a, b) in enumerate(zip(greedy, want)) if a != b), 12)
    assert k >= 6
    outs = []
    for seed in (3, 3, 4):
        assert G.main(["--model", folder, "--prompt-ids", "5,6,7", "--n-predict", "12", "--temp", "1.5", "--top-k", "5", "--seed", str(seed)]) == 0
        outs.append(capsys.readouterr().out.strip())
    assert outs[0] == outs[1] and len(outs[0].split(",")) == 12
    # every sampled token lies in the top 5 of the logits the oracle gives for the tokens before it
    toks = [int(t) for t in outs[0].split(",")]
    lg = O.run(m, [5, 6, 7] + toks)
    for i, t in enumerate(toks):
        assert t in np.argsort(-lg[2 + i])[:6], i


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_trace_runner_replays_steps_and_writes_the_wanted_rows(tmp_path, dtype):
    """bin/trace_run as a program: requests one after the other, portions of changing size, rows only where asked, a line per step; against the oracle"""
    import subprocess
    import sys
    m = small_model(seed=81, layers=VARIANTS["other_sizes"], width=40)
    folder, out = str(tmp_path / "model"), str(tmp_path / "out")
    O.write_model(folder, m["config"], {k: v.astype(np.float32) for k, v in m["tensors"].items()})
    rng = np.random.default_rng(5)
    a, b = [int(t) for t in rng.integers(0, 97, 41)], [int(t) for t in rng.integers(0, 97, 9)]
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
        got = np.fromfile(os.path.join(out, "%d.f32" % k), "<f4").reshape(-1, 97)
        assert got.shape == w.shape and logit_err(got, w).max() < TOL[dtype == "float32"], k
