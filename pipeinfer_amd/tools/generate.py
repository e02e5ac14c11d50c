"""Generate a continuation of token ids with any model the engine loads (a GGUF file, or a folder with config.json + model.safetensors):

    python -m pipeinfer_amd.tools.generate --model PATH --prompt-ids 1,2,3 --n-predict 32 [--temp 0.8 --top-k 40 --top-p 0.95 --seed 1] [--float32]

The prompt goes through llama_decode in passes of n_batch tokens, every new token through one more pass; tokens are chosen by the engine's own samplers
(llama_sample_top_k / _top_p / _temp / _token, or the device-side arg-max with --temp 0).  Prints the generated ids, one line."""
import argparse
import ctypes as C
import sys

import numpy as np

from .. import llama as LL


class TokenData(C.Structure):
    _fields_ = [("id", C.c_int32), ("logit", C.c_float), ("p", C.c_float)]


class TokenDataArray(C.Structure):
    _fields_ = [("data", C.POINTER(TokenData)), ("size", C.c_size_t), ("sorted", C.c_bool)]


def sample(lib, ctx, logits, temp, top_k, top_p):
    """one token from a row of logits through the llama.h samplers"""
    n = len(logits)
    arr = (TokenData * n)()
    ids = np.arange(n, dtype=np.int32)
    view = np.ctypeslib.as_array(C.cast(arr, C.POINTER(C.c_int32)), shape=(n, 3))
    view[:, 0] = ids
    view[:, 1] = np.ascontiguousarray(logits, np.float32).view(np.int32)
    view[:, 2] = 0
    cands = TokenDataArray(arr, n, False)
    vp = C.c_void_p
    lib.llama_sample_top_k.argtypes = [vp, C.POINTER(TokenDataArray), C.c_int, C.c_size_t]
    lib.llama_sample_top_p.argtypes = [vp, C.POINTER(TokenDataArray), C.c_float, C.c_size_t]
    lib.llama_sample_temp.argtypes = [vp, C.POINTER(TokenDataArray), C.c_float]
    lib.llama_sample_token.argtypes = [vp, C.POINTER(TokenDataArray)]
    if top_k > 0:
        lib.llama_sample_top_k(ctx.h, C.byref(cands), top_k, 1)
    if top_p < 1.0:
        lib.llama_sample_top_p(ctx.h, C.byref(cands), top_p, 1)
    lib.llama_sample_temp(ctx.h, C.byref(cands), temp)
    return int(lib.llama_sample_token(ctx.h, C.byref(cands)))


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", required=True)
    ap.add_argument("--prompt-ids", required=True, help="comma-separated token ids")
    ap.add_argument("--n-predict", type=int, default=32)
    ap.add_argument("--n-ctx", type=int, default=0, help="cells of the cache (default: prompt + n-predict)")
    ap.add_argument("--n-batch", type=int, default=512)
    ap.add_argument("--temp", type=float, default=0.0)
    ap.add_argument("--top-k", type=int, default=40)
    ap.add_argument("--top-p", type=float, default=0.95)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--float32", action="store_true", help="dense-weight models: every product in fp32")
    a = ap.parse_args(argv)
    prompt = [int(t) for t in a.prompt_ids.split(",") if t.strip()]
    model = LL.Model(a.model)
    n_ctx = a.n_ctx or max(32, len(prompt) + a.n_predict + 1)
    ctx = LL.Context(model, n_ctx=n_ctx, n_batch=min(a.n_batch, n_ctx))
    if a.float32:
        ctx.set_precision(True)
    lib = ctx.lib
    lib.llama_set_rng_seed.argtypes = [C.c_void_p, C.c_uint32]
    lib.llama_set_rng_seed(ctx.h, a.seed)
    if a.temp <= 0.0:
        out = ctx.generate(prompt, a.n_predict)
    else:
        out, pos = [], len(prompt)
        logits = ctx.feed(prompt, 0, 0)[-1]
        for _ in range(a.n_predict):
            tok = sample(lib, ctx, logits, a.temp, a.top_k, a.top_p)
            out.append(tok)
            logits = ctx.decode([tok], [pos], [[0]])[0]
            pos += 1
    print(",".join(str(t) for t in out))
    ctx.free()
    model.free()
    return 0


if __name__ == "__main__":
    sys.exit(main())
