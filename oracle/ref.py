"""TEST INFRASTRUCTURE ONLY: ctypes binding of oracle/libwgpt_oracle.so.

Thin numpy-in / numpy-out wrappers around the C restatement of the reference's
WGSL kernels (oracle/wgpt_oracle.c, which cites the reference per function).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libwgpt_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()
_f = C.POINTER(C.c_float)
_i = C.POINTER(C.c_int32)


def _fp(a):
    return None if a is None else a.ctypes.data_as(_f)


def _ip(a):
    return None if a is None else a.ctypes.data_as(_i)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _i32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.int32)


class _Layer(C.Structure):
    _fields_ = [(n, _f) for n in ("ln1_g", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b",
                                  "ln2_g", "ln2_b", "fc_w", "fc_b", "fc2_w", "fc2_b")] + \
               [(n, _i) for n in ("attn_q", "proj_q", "fc_q", "fc2_q")] + \
               [(n, _f) for n in ("attn_s", "proj_s", "fc_s", "fc2_s")]


class _Model(C.Structure):
    _fields_ = [("n_layer", C.c_int), ("n_head", C.c_int), ("n_embd", C.c_int), ("n_ctx", C.c_int),
                ("vocab_size", C.c_int), ("wte", _f), ("wpe", _f), ("lnf_g", _f), ("lnf_b", _f),
                ("layers", C.POINTER(_Layer))]


_lib.ref_quantize_global.restype = C.c_float
_lib.ref_get_threads.restype = C.c_int
_lib.ref_forward.restype = C.c_int


def set_threads(n):
    _lib.ref_set_threads(C.c_int(int(n)))


def get_threads():
    return int(_lib.ref_get_threads())


def matmul_bias(A, B, bias=None):
    A, B, bias = _f32(A), _f32(B), _f32(bias)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    out = np.empty((M, N), np.float32)
    _lib.ref_matmul_bias(M, N, K, _fp(A), _fp(B), _fp(bias), _fp(out))
    return out


def residual(a, b):
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    M, N = a.shape
    _lib.ref_residual(M, N, _fp(a), _fp(b), _fp(out))
    return out


def layernorm_stats(x):
    x = _f32(x)
    M, N = x.shape
    st = np.empty((M, 2), np.float32)
    _lib.ref_layernorm_stats(M, N, _fp(x), _fp(st))
    return st


def layernorm(x, gamma, beta):
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    M, N = x.shape
    out = np.empty_like(x)
    _lib.ref_layernorm(M, N, _fp(x), _fp(gamma), _fp(beta), _fp(out))
    return out


def softmax(x):
    x = _f32(x)
    M, N = x.shape
    out = np.empty_like(x)
    _lib.ref_softmax(M, N, _fp(x), _fp(out))
    return out


def gelu(x):
    x = _f32(x)
    M, N = x.shape
    out = np.empty_like(x)
    _lib.ref_gelu(M, N, _fp(x), _fp(out))
    return out


def embed(idx, wte, wpe):
    idx, wte, wpe = _i32(idx), _f32(wte), _f32(wpe)
    T, d = idx.shape[0], wte.shape[1]
    out = np.empty((T, d), np.float32)
    _lib.ref_embed(_ip(idx), T, d, _fp(wte), _fp(wpe), _fp(out))
    return out


def deembed(x, wte):
    x, wte = _f32(x), _f32(wte)
    T, d = x.shape
    V = wte.shape[0]
    out = np.empty(V, np.float32)
    _lib.ref_deembed(d, V, T, _fp(x), _fp(wte), _fp(out))
    return out


def format_q(Q, hs):
    Q = _f32(Q)
    T, d = Q.shape
    out = np.empty((d // hs, T, hs), np.float32)
    _lib.ref_format_q(T, d, hs, _fp(Q), _fp(out))
    return out


def attn_weights(Qf, Kmat, scale):
    Qf, Kmat = _f32(Qf), _f32(Kmat)
    H, T, hs = Qf.shape
    out = np.empty((H * T, T), np.float32)
    _lib.ref_attn_weights(T, H, hs, C.c_float(scale), _fp(Qf), _fp(Kmat), _fp(out))
    return out


def attn_values(P, V, hs):
    P, V = _f32(P), _f32(V)
    T, d = V.shape
    out = np.empty((T, d), np.float32)
    _lib.ref_attn_values(T, d, hs, _fp(P), _fp(V), _fp(out))
    return out


def attention(x, Wq, bq, Wk, bk, Wv, bv, Wo, bo, n_head, scale=None, return_kv=False):
    arrs = [_f32(a) for a in (x, Wq, bq, Wk, bk, Wv, bv, Wo, bo)]
    T, d = arrs[0].shape
    hs = d // n_head
    if scale is None:
        scale = np.float32(1.0 / np.sqrt(hs))
    out = np.empty((T, d), np.float32)
    Ko = np.empty((T, d), np.float32)
    Vo = np.empty((T, d), np.float32)
    _lib.ref_attention_kv(T, d, C.c_float(scale), n_head, hs, *[_fp(a) for a in arrs], _fp(out), _fp(Ko), _fp(Vo))
    return (out, Ko, Vo) if return_kv else out


def dequant_i8(Bq, scale, N):
    Bq, scale = _i32(Bq), _f32(scale)
    K = Bq.shape[0]
    out = np.empty((K, N), np.float32)
    _lib.ref_dequant_i8(K, N, _ip(Bq), _fp(scale), _fp(out))
    return out


def matmul_i8(A, Bq, scale, bias=None):
    A, Bq, scale, bias = _f32(A), _i32(Bq), _f32(scale), _f32(bias)
    M, K = A.shape
    N = scale.shape[0]
    out = np.empty((M, N), np.float32)
    _lib.ref_matmul_i8(M, N, K, _fp(A), _ip(Bq), _fp(scale), _fp(bias), _fp(out))
    return out


def quantize_global(w):
    w = _f32(w).ravel()
    packed = np.empty((w.size + 3) // 4, np.int32)
    absmax = _lib.ref_quantize_global(w.size, _fp(w), _ip(packed))
    return packed, np.float32(absmax)


def dequantize_js(packed, absmax, count):
    packed = _i32(packed)
    out = np.empty(count, np.float32)
    _lib.ref_dequantize_js(count, _ip(packed), C.c_float(absmax), _fp(out))
    return out


def sample_topk(logits, top_k, temperature, u):
    """(id, ids[k], probs[k]) of model.js:81-85 with `u` standing for Math.random()."""
    logits = _f32(logits).ravel()
    k = min(int(top_k), logits.size)
    ids = np.empty(k, np.int32)
    probs = np.empty(k, np.float64)
    _lib.ref_sample_topk.restype = C.c_int
    chosen = _lib.ref_sample_topk(logits.size, int(top_k), C.c_double(temperature), C.c_double(u), _fp(logits), _ip(ids),
                                  probs.ctypes.data_as(C.POINTER(C.c_double)))
    return int(chosen), ids, probs


LAYER_F32 = ("ln1_g", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b", "ln2_g", "ln2_b", "fc_w", "fc_b", "fc2_w", "fc2_b")
LAYER_I8 = ("attn", "proj", "fc", "fc2")


def forward(params, weights, tokens, want_taps=False, want_kv=False):
    """GPT.run() on the CPU oracle.

    params: dict n_layer, n_head, n_embd, n_ctx, vocab_size.
    weights: dict wte, wpe, lnf_g, lnf_b, layers=[dict of LAYER_F32 names, and for the
    int8 variant {attn,proj,fc,fc2}_q (packed int32 [K,N/4]) and _s (scale [N])].
    Returns logits[V] (and taps [(2+6L),T,d], kv [L,2,T,d] when asked).
    """
    L, d, V = params["n_layer"], params["n_embd"], params["vocab_size"]
    tokens = _i32(tokens)
    T = tokens.shape[0]
    keep = []
    layers = (_Layer * L)()
    for li, lw in enumerate(weights["layers"]):
        for n in LAYER_F32:
            a = _f32(lw.get(n))
            keep.append(a)
            setattr(layers[li], n, _fp(a))
        for n in LAYER_I8:
            q, s = _i32(lw.get(n + "_q")), _f32(lw.get(n + "_s"))
            keep += [q, s]
            setattr(layers[li], n + "_q", _ip(q))
            setattr(layers[li], n + "_s", _fp(s))
    m = _Model()
    m.n_layer, m.n_head, m.n_embd, m.n_ctx, m.vocab_size = L, params["n_head"], d, params["n_ctx"], V
    top = [_f32(weights[n]) for n in ("wte", "wpe", "lnf_g", "lnf_b")]
    m.wte, m.wpe, m.lnf_g, m.lnf_b = [_fp(a) for a in top]
    m.layers = layers
    logits = np.empty(V, np.float32)
    taps = np.empty((2 + 6 * L, T, d), np.float32) if want_taps else None
    kv = np.empty((L, 2, T, d), np.float32) if want_kv else None
    rc = _lib.ref_forward(C.byref(m), _ip(tokens), T, _fp(logits), _fp(taps), _fp(kv))
    if rc != 0:
        raise ValueError("ref_forward: bad arguments")
    out = [logits]
    if want_taps:
        out.append(taps)
    if want_kv:
        out.append(kv)
    return out[0] if len(out) == 1 else tuple(out)


def tap_names(n_layer):
    """Names of the activation taps, other/validation/validation.js:183-205."""
    names = ["tok_pos_emb"]
    for i in range(n_layer):
        names += [f"block{i}_{s}" for s in ("ln1", "attn", "r1", "ln2", "mlp", "r2")]
    return names + ["ln_f"]
