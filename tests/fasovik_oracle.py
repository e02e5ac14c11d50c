"""Plain, slow restatement of the Fasovik design in numpy (float64), one function per mechanism: the oracle the engine's kernels are
held to.  It shares no code with the product path: token by token, head by head, no cache tricks, no fused steps.

A model is a dict: {"config": <the config.json dictionary>, "tensors": {name: float64 array}}.

Notation.  A layer reads the residual x, runs a sublayer on x itself and adds m * N1(sublayer(x)), N1(y) = y / sqrt(mean(y^2) + eps) * (1 + w):
the norm sits on the sublayer's OUTPUT.  Mixers:
  lightning          per head a matrix state  S <- lambda_h * S + k v^T,  o = S^T q  with q, k, v = silu(projection); heads concatenated, RMS-normed as
                     one vector (plain weight), gated by sigmoid(W_g h), projected by W_o
  latent_attention   keys and values are up-projections of one shared low-rank latent c = N(W_dkv h) (plain weight); no positions; causal; the softmax
                     denominator carries one extra term exp(sink_h) that has no value
Feed-forward: a mixture of experts whose router also owns "identity experts" that return their input.
"""
import json
import struct

import numpy as np


# ---- files ------------------------------------------------------------------------------------------------------------------
def bf16_round(a):
    """float32 values rounded to the nearest bfloat16 (ties to even), returned as float32"""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def write_model(folder, config, tensors):
    """config.json + model.safetensors: float tensors as bfloat16 (values must already be bfloat16-representable), integer tensors as int32"""
    import os
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    head, blobs, at = {}, [], 0
    for name, t in tensors.items():
        if np.issubdtype(np.asarray(t).dtype, np.integer):
            raw, dt = np.asarray(t, np.int32).tobytes(), "I32"
        else:
            u = np.ascontiguousarray(t, np.float32).view(np.uint32)
            assert not (u & 0xFFFF).any(), name
            raw, dt = (u >> 16).astype(np.uint16).tobytes(), "BF16"
        head[name] = {"dtype": dt, "shape": list(np.shape(t)), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    h = json.dumps(head).encode()
    h += b" " * (-len(h) % 8)
    with open(os.path.join(folder, "model.safetensors"), "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + b"".join(blobs))


def read_model(folder):
    import os
    with open(os.path.join(folder, "config.json")) as f:
        config = json.load(f)
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        n, = struct.unpack("<Q", f.read(8))
        head = json.loads(f.read(n))
        data = f.read()
    tensors = {}
    for name, d in head.items():
        if name == "__metadata__":
            continue
        a, b = d["data_offsets"]
        if d["dtype"] == "BF16":
            t = (np.frombuffer(data[a:b], np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif d["dtype"] == "F32":
            t = np.frombuffer(data[a:b], np.float32).astype(np.float64)
        elif d["dtype"] == "I32":
            t = np.frombuffer(data[a:b], np.int32)
        else:
            raise ValueError(d["dtype"])
        tensors[name] = t.reshape(d["shape"])
    return {"config": config, "tensors": tensors}


# ---- small functions --------------------------------------------------------------------------------------------------------
def rms(x, eps):
    return x / np.sqrt(np.mean(x * x) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softmax(z):
    e = np.exp(z - z.max())
    return e / e.sum()


# ---- mechanisms (each for ONE token, with whatever the sequence has left behind) ---------------------------------------------
def lightning_step(T, p, mix, eps, h, state):
    """state: [heads][dim][vdim] of this layer and sequence (zeros at the start); returns the mixer's output, updates state in place"""
    H, D, V = mix["heads"], mix["dim"], mix["vdim"]
    q = silu(T[p + "mix.q"] @ h).reshape(H, D)
    k = silu(T[p + "mix.k"] @ h).reshape(H, D)
    v = silu(T[p + "mix.v"] @ h).reshape(H, V)
    o = np.zeros((H, V))
    for i in range(H):
        state[i] = mix["decay"][i] * state[i] + np.outer(k[i], v[i])
        o[i] = state[i].T @ q[i]
    y = rms(o.reshape(-1), eps) * T[p + "mix.norm"] * sigmoid(T[p + "mix.g"] @ h)
    return T[p + "mix.o"] @ y


def latent_attention_step(T, p, mix, eps, h, latents):
    """latents: list of the latent vectors of the earlier tokens of this layer and sequence; this token's is appended"""
    H, D, V = mix["heads"], mix["dim"], mix["vdim"]
    q = (T[p + "mix.q"] @ h).reshape(H, D)
    latents.append(rms(T[p + "mix.dkv"] @ h, eps) * T[p + "mix.dkv.norm"])
    C = np.stack(latents)                                   # [tokens so far][kv_rank]
    K = (C @ T[p + "mix.uk"].T).reshape(len(C), H, D)
    Vv = (C @ T[p + "mix.uv"].T).reshape(len(C), H, V)
    out = np.zeros((H, V))
    for i in range(H):
        s = K[:, i, :] @ q[i] * mix["scale"]
        m = max(s.max(), T[p + "mix.sink"][i])
        e = np.exp(s - m)
        out[i] = (e / (e.sum() + np.exp(T[p + "mix.sink"][i] - m))) @ Vv[:, i, :]
    return T[p + "mix.o"] @ out.reshape(-1)


def moe_route(T, p, mlp, h):
    """(chosen router outputs, their weights); outputs >= experts are identity experts"""
    r = mlp["router"]
    s = softmax(T[p + "mlp.router"] @ h)
    choice = s + T[p + "mlp.correction"]
    order = sorted(range(len(s)), key=lambda e: (-choice[e], e))[: r["top"]]
    return order, [s[e] for e in order]


def moe(T, p, mlp, h):
    n_exp = mlp["router"]["experts"]
    out = np.zeros_like(h)
    for e, w in zip(*moe_route(T, p, mlp, h)):
        if e >= n_exp:
            out += w * h
        else:
            out += w * (T[p + "mlp.e%d.down" % e] @ np.maximum(T[p + "mlp.e%d.up" % e] @ h, 0.0) ** 2)
    return out


# ---- the model ----------------------------------------------------------------------------------------------------------------
class Sequence:
    """what one sequence has left behind: per layer a state matrix or a list of latents"""

    def __init__(self, model):
        self.per_layer = []
        for L in model["config"]["layers"]:
            m = L["mixer"]
            self.per_layer.append(np.zeros((m["heads"], m["dim"], m["vdim"])) if L["type"] == "lightning" else [])


def step(model, seq, token, layers_out=None):
    """one token through the model; returns its logits (float64)"""
    cfg, T = model["config"], model["tensors"]
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = T["embed"][token] * cfg["embedding"]["scale"]
    for i, L in enumerate(cfg["layers"]):
        j = i
        while "weights_of" in cfg["layers"][j]:               # (a borrowed layer may itself borrow)
            j = cfg["layers"][j]["weights_of"]
        p = "l%d." % j
        if L["type"] == "lightning":
            y = lightning_step(T, p, L["mixer"], eps, x, seq.per_layer[i])
        elif L["type"] == "latent_attention":
            y = latent_attention_step(T, p, L["mixer"], eps, x, seq.per_layer[i])
        else:
            raise ValueError(L["type"])
        x = x + m * rms(y, eps) * (1.0 + T[p + "norm1"])
        if L.get("mlp") is not None:
            x = x + m * rms(moe(T, p, L["mlp"], x), eps) * (1.0 + T[p + "norm2"])
        if layers_out is not None:
            layers_out.append(x.copy())
    return T["embed"] @ (rms(x, eps) * (1.0 + T["final.norm"]))


def run(model, tokens, layers=False):
    """logits [len(tokens)][vocab] of one sequence from its start (and the residual stream [layer][token][width] with layers=True)"""
    seq, out, res = Sequence(model), [], []
    for t in tokens:
        lo = [] if layers else None
        out.append(step(model, seq, int(t), lo))
        if layers:
            res.append(lo)
    if layers:
        return np.array(out), np.transpose(np.array(res), (1, 0, 2))
    return np.array(out)


def greedy(model, prompt, n):
    seq, toks = Sequence(model), list(prompt)
    for t in toks[:-1]:
        step(model, seq, int(t))
    for _ in range(n):
        toks.append(int(np.argmax(step(model, seq, toks[-1]))))
    return toks[len(prompt):]


# ---- random models --------------------------------------------------------------------------------------------------------------
def random_model(rng, vocab, width, layers, eps=1e-5, residual_mult=0.4, embed_scale=2.0):
    """layers: list of dicts {"type", "mixer": {...sizes...}, "mlp": {"ff", "experts", "identity", "top"} or None, optional "weights_of"};
    returns a model whose float tensors are bfloat16-representable"""
    def w(*shape, s=None):
        s = s if s is not None else 1.0 / np.sqrt(shape[-1])
        return bf16_round(rng.standard_normal(shape).astype(np.float32) * s).astype(np.float64)
    T = {"embed": w(vocab, width, s=0.5), "final.norm": w(width, s=0.2)}
    cfg_layers = []
    for i, L in enumerate(layers):
        mix = dict(L["mixer"])
        entry = {"type": L["type"], "mixer": mix, "mlp": None}
        if L.get("mlp"):
            f = L["mlp"]
            entry["mlp"] = {"kind": "moe", "expert": {"ff": f["ff"]}, "router": {"experts": f["experts"], "identity": f["identity"], "top": f["top"]}}
        if "weights_of" in L:
            entry["weights_of"] = L["weights_of"]
            cfg_layers.append(entry)
            continue
        p = "l%d." % i
        H, D, V = mix["heads"], mix["dim"], mix["vdim"]
        T[p + "norm1"] = w(width, s=0.2)
        if L["type"] == "lightning":
            for n, rows in (("q", H * D), ("k", H * D), ("v", H * V), ("g", H * V)):
                T[p + "mix." + n] = w(rows, width)
            T[p + "mix.o"] = w(width, H * V)
            T[p + "mix.norm"] = w(H * V, s=0.3) + 1.0
            T[p + "mix.norm"] = bf16_round(T[p + "mix.norm"].astype(np.float32)).astype(np.float64)
        else:
            R = mix["kv_rank"]
            T[p + "mix.q"] = w(H * D, width, s=2.0 / np.sqrt(width))
            T[p + "mix.dkv"] = w(R, width)
            T[p + "mix.dkv.norm"] = bf16_round((rng.standard_normal(R) * 0.3 + 1.0).astype(np.float32)).astype(np.float64)
            T[p + "mix.uk"] = w(H * D, R, s=2.0 / np.sqrt(R))
            T[p + "mix.uv"] = w(H * V, R)
            T[p + "mix.sink"] = w(H, s=1.0)
            T[p + "mix.o"] = w(width, H * V)
        if L.get("mlp"):
            f = L["mlp"]
            T[p + "norm2"] = w(width, s=0.2)
            for e in range(f["experts"]):
                T[p + "mlp.e%d.up" % e] = w(f["ff"], width)
                T[p + "mlp.e%d.down" % e] = w(width, f["ff"])
            T[p + "mlp.router"] = w(f["experts"] + f["identity"], width, s=2.0 / np.sqrt(width))
            T[p + "mlp.correction"] = w(f["experts"] + f["identity"], s=0.05)
        cfg_layers.append(entry)
    config = {"architecture": "Fasovik", "vocab": vocab, "width": width, "embedding": {"scale": embed_scale}, "norm": {"eps": eps},
              "residual_mult": residual_mult, "layers": cfg_layers}
    return {"config": config, "tensors": T}
