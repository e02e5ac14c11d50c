"""Plain, slow restatement of the Vikarax design in numpy (float64), one function per mechanism, token by token: the oracle the engine's kernels are held to.
It shares no code with the product path (file reading and bfloat16 rounding come from the other oracle of this folder, which is test infrastructure too).

A model is {"config": <the config.json dictionary>, "tensors": {name: float64 array}}.

Notation.  LN_a(y) = (y - mean y) / sqrt(var y + eps) * w_a + b_a (var = mean of squared deviations), R(y) = y / sqrt(mean(y^2) + eps).
A layer i:   x' = x + LN_1b(mixer(LN_1(x)));   x'' = x' + LN_2b(ff(LN_2(x')))  (without a feed-forward x'' = x');   X_(i+1) = x'';
             what the next layer (or the output) reads = sum_(j <= i+1) dwa_i[j] X_j, X_0 the embedding row.
Mixer:       left_scale * attention(h) + right_scale * recurrence(h), both on the same h.
  attention   H query heads over G key/value heads; q, k: per head R(.) * w (one weight vector for all heads), then the first `dims` dimensions rotated by the position
              (dimension i with i + dims/2, angle p * base^(-2i/dims)); v: per head R(.), no weight; weight of key j for query i = sigmoid(q.k * scale + pb_h) when j <= i lies
              in the same block of `size` positions, else 0; nothing is normalised; head output * sigmoid(W_g h)_h; W_o.
  recurrence  W_in h = [z | x | B | C | dt]; (x, B, C) through a causal per-channel convolution of `conv` taps + bias, then silu; dt = softplus(dt + dt_bias);
              per head S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x (B, C of the head's group); (y * silu(z)) R-normed in `norm_groups` parts, * w; W_o.
Feed-forward: dense  W_down relu(W_up h)^2;   routed  s = sigmoid(W_r h), groups of consecutive experts ranked by top1 + top2 of s, members of the `keep` highest-ranked groups compete, the `top` highest s win
              with weight s (as it is); expert = W_down (silu(W_gate h) * W_up h); a shared expert of the same form is added for every token.
Output:      cap * tanh((W_head LN_f(x)) / cap).
"""
import numpy as np

from tests.fasovik_oracle import bf16_round, read_model, write_model  # noqa: F401  (files and rounding: shared test infrastructure)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def layer_norm(y, w, b, eps):
    d = y - y.mean()
    return d / np.sqrt((d * d).mean() + eps) * w + b


def unit_rms(y, eps):
    return y / np.sqrt((y * y).mean() + eps)


def rotate(vec, pos, dims, base):
    """the first `dims` entries of vec, in pairs (i, i + dims/2), turned by pos * base^(-2i/dims)"""
    out = vec.copy()
    half = dims // 2
    for i in range(half):
        a = pos * base ** (-2.0 * i / dims)
        u, v = vec[i], vec[i + half]
        out[i], out[i + half] = u * np.cos(a) - v * np.sin(a), v * np.cos(a) + u * np.sin(a)
    return out


# ---- the two branches of the mixer ------------------------------------------------------------------------------------------
def attention_step(T, p, c, eps, h, pos, keys, values):
    """one token of the attention branch; keys / values: what the sequence has cached so far [(position, [G][dim]), ...]; this token's are appended"""
    H, G, D, V = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    rot = c.get("rot") or {"dims": 0, "base": 1.0}
    q = (T[p + "q"] @ h).reshape(H, D)
    k = (T[p + "k"] @ h).reshape(G, D)
    v = (T[p + "v"] @ h).reshape(G, V)
    q = np.stack([rotate(unit_rms(q[i], eps) * T[p + "q.norm"], pos, rot["dims"], rot["base"]) for i in range(H)])
    k = np.stack([rotate(unit_rms(k[i], eps) * T[p + "k.norm"], pos, rot["dims"], rot["base"]) for i in range(G)])
    v = np.stack([unit_rms(v[i], eps) for i in range(G)])
    keys.append((pos, k))
    values.append(v)
    size = (c.get("mask") or {}).get("size")
    gate = sigmoid(T[p + "g"] @ h)
    out = np.zeros((H, V))
    for i in range(H):
        g = i // (H // G)
        for (pj, kj), vj in zip(keys, values):
            if pj > pos or (size and pj // size != pos // size):
                continue
            out[i] += sigmoid(q[i] @ kj[g] * c["scale"] + T[p + "pb"][i]) * vj[g]
        out[i] *= gate[i]
    return T[p + "o"] @ out.reshape(-1)


def recurrence_step(T, p, c, eps, h, state):
    """one token of the recurrence; state = {"S": [heads][N][vdim], "tail": the last conv - 1 inputs of the convolution, oldest first}"""
    Hn, P, N, G, taps = c["heads"], c["vdim"], c["state"], c["groups"], c["conv"]
    inner = Hn * P
    u = T[p + "in"] @ h
    z, xbc, dt = u[:inner], u[inner:2 * inner + 2 * G * N], u[2 * inner + 2 * G * N:]
    window = state["tail"] + [xbc]                               # the current token's input is weighed by the last tap
    conv = T[p + "conv.b"].copy()
    for l in range(taps):
        conv += T[p + "conv"][:, l] * window[l]
    state["tail"] = window[1:]
    xbc = silu(conv)
    x, B, Cm = xbc[:inner].reshape(Hn, P), xbc[inner:inner + G * N].reshape(G, N), xbc[inner + G * N:].reshape(G, N)
    dt = softplus(dt + T[p + "dt_bias"])
    y = np.zeros((Hn, P))
    for i in range(Hn):
        g = i // (Hn // G)
        state["S"][i] = np.exp(-np.exp(T[p + "A_log"][i]) * dt[i]) * state["S"][i] + dt[i] * np.outer(B[g], x[i])
        y[i] = state["S"][i].T @ Cm[g] + T[p + "D"][i] * x[i]
    y = y.reshape(-1) * silu(z)
    parts = c.get("norm_groups", 1)
    y = np.concatenate([unit_rms(part, eps) for part in y.reshape(parts, -1)]) * T[p + "norm"]
    return T[p + "o"] @ y


def new_recurrence_state(c):
    return {"S": np.zeros((c["heads"], c["state"], c["vdim"])), "tail": [np.zeros(c["heads"] * c["vdim"] + 2 * c["groups"] * c["state"]) for _ in range(c["conv"] - 1)]}


# ---- feed-forward ------------------------------------------------------------------------------------------------------------
def gated_expert(T, p, h):
    return T[p + "down"] @ (silu(T[p + "gate"] @ h) * (T[p + "up"] @ h))


def route(T, p, mlp, h):
    """(indices, weights) of the experts a token uses: group-limited choice by sigmoid score, lowest index on a tie"""
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    s = sigmoid(T[p + "router"] @ h)
    per = E // groups["count"]
    gscore = [np.sort(s[g * per:(g + 1) * per])[::-1][:2].sum() for g in range(groups["count"])]
    kept = sorted(range(groups["count"]), key=lambda g: (-gscore[g], g))[:groups["keep"]]
    cand = [e for e in range(E) if e // per in kept]
    chosen = sorted(cand, key=lambda e: (-s[e], e))[:top]
    return chosen, [s[e] for e in chosen]


def feed_forward(T, p, mlp, h):
    if mlp["kind"] == "dense":
        return T[p + "down"] @ (np.maximum(T[p + "up"] @ h, 0.0) ** 2)
    idx, w = route(T, p, mlp, h)
    out = sum(wi * gated_expert(T, p + "e%d." % e, h) for e, wi in zip(idx, w))
    if mlp.get("shared"):
        out = out + gated_expert(T, p + "shared.", h)
    return out


# ---- the model, token by token ---------------------------------------------------------------------------------------------
class Sequence:
    def __init__(self, model):
        L = model["config"]["layers"]
        self.keys, self.values = [[] for _ in L], [[] for _ in L]
        self.rec = [new_recurrence_state(l["mixer"]["right"]) for l in L]
        self.n = 0


def step(model, seq, token, layers_out=None):
    cfg, T = model["config"], model["tensors"]
    eps = cfg["norm"]["eps"]
    x = T["embed"][token].copy()
    history = [x]
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        m = L["mixer"]
        h = layer_norm(x, T[p + "norm1"], T[p + "norm1.b"], eps)
        mix = m["left_scale"] * attention_step(T, p + "mix.left.", m["left"], eps, h, seq.n, seq.keys[i], seq.values[i]) \
            + m["right_scale"] * recurrence_step(T, p + "mix.right.", m["right"], eps, h, seq.rec[i])
        x = x + layer_norm(mix, T[p + "norm1b"], T[p + "norm1b.b"], eps)
        if L.get("mlp"):
            h = layer_norm(x, T[p + "norm2"], T[p + "norm2.b"], eps)
            x = x + layer_norm(feed_forward(T, p + "mlp.", L["mlp"], h), T[p + "norm2b"], T[p + "norm2b.b"], eps)
        history.append(x)
        x = sum(T[p + "dwa"][j] * history[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x.copy())
    seq.n += 1
    z = T["head"] @ layer_norm(x, T["final.norm"], T["final.norm.b"], eps)
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z


def run(model, tokens):
    seq = Sequence(model)
    return np.stack([step(model, seq, t) for t in tokens])


def greedy(model, prompt, n):
    seq = Sequence(model)
    for t in prompt[:-1]:
        step(model, seq, t)
    out, last = [], prompt[-1]
    for _ in range(n):
        last = int(np.argmax(step(model, seq, last)))
        out.append(last)
    return out


# ---- random models ---------------------------------------------------------------------------------------------------------
def parallel_layer(heads=3, kv_heads=1, dim=8, vdim=6, chunk=7, rot_dims=4, rot_base=50.0, scale=0.4, r_heads=4, r_vdim=5, state=6, groups=2, conv=3, norm_groups=2,
                   left_scale=0.7, right_scale=1.1, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        left["mask"] = {"size": chunk}
    if rot_dims:
        left["rot"] = {"dims": rot_dims, "base": rot_base}
    right = {"heads": r_heads, "vdim": r_vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}, "mlp": mlp}


def dense_mlp(ff):
    return {"kind": "dense", "ff": ff}


def routed_mlp(experts, top, ff, count=1, keep=1, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def random_model(rng, vocab, width, layers, eps=1e-5, softcap=12.0):
    """bfloat16-representable random tensors, scaled so that activations stay of order one through the layers"""
    def w(*shape, s=None):
        s = s if s is not None else 1.0 / np.sqrt(shape[-1])
        return bf16_round((rng.standard_normal(shape) * s).astype(np.float32)).astype(np.float64)

    def around(c, *shape, s=0.2):
        return bf16_round((c + rng.standard_normal(shape) * s).astype(np.float32)).astype(np.float64)
    T = {"embed": w(vocab, width, s=1.0), "head": w(vocab, width), "final.norm": around(1.0, width), "final.norm.b": w(width, s=0.1)}
    for i, L in enumerate(layers):
        p = "l%d." % i
        a, r = L["mixer"]["left"], L["mixer"]["right"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if L.get("mlp") else ()):
            T[p + n], T[p + n + ".b"] = around(1.0, width), w(width, s=0.1)
        T[p + "dwa"] = around(1.0 / (i + 2), i + 2, s=0.15)
        q = p + "mix.left."
        T[q + "q"], T[q + "k"], T[q + "v"] = w(a["heads"] * a["dim"], width), w(a["kv_heads"] * a["dim"], width), w(a["kv_heads"] * a["vdim"], width)
        T[q + "q.norm"], T[q + "k.norm"] = around(1.0, a["dim"]), around(1.0, a["dim"])
        T[q + "pb"], T[q + "g"], T[q + "o"] = w(a["heads"], s=1.0), w(a["heads"], width), w(width, a["heads"] * a["vdim"])
        q = p + "mix.right."
        inner, gn = r["heads"] * r["vdim"], r["groups"] * r["state"]
        T[q + "in"] = w(2 * inner + 2 * gn + r["heads"], width)
        T[q + "conv"], T[q + "conv.b"] = w(inner + 2 * gn, r["conv"], s=0.5), w(inner + 2 * gn, s=0.2)
        T[q + "dt_bias"], T[q + "A_log"], T[q + "D"] = w(r["heads"], s=0.7), around(-0.5, r["heads"], s=0.8), around(1.0, r["heads"], s=0.3)
        T[q + "norm"], T[q + "o"] = around(1.0, inner), w(width, inner)
        mlp = L.get("mlp")
        if mlp and mlp["kind"] == "dense":
            T[p + "mlp.up"], T[p + "mlp.down"] = w(mlp["ff"], width), w(width, mlp["ff"])
        elif mlp:
            T[p + "mlp.router"] = w(mlp["router"]["experts"], width, s=2.0 / np.sqrt(width))
            names = ["e%d" % e for e in range(mlp["router"]["experts"])] + (["shared"] if mlp.get("shared") else [])
            for n in names:
                ff = mlp["shared"]["ff"] if n == "shared" else mlp["expert"]["ff"]
                T[p + "mlp.%s.gate" % n], T[p + "mlp.%s.up" % n], T[p + "mlp.%s.down" % n] = w(ff, width), w(ff, width), w(width, ff)
    cfg = {"architecture": "Vikarax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_softcap": softcap, "layers": layers}
    return {"config": cfg, "tensors": T}
