"""Weight-only int8 quantisation of a linear weight: the host side of other/int8-gemm.js.

`quantizeMatrix` is the reference's function of the same name (other/int8-gemm.js:25-46)
with the one change its own header asks for (line 4: "adjust the absmax from being a global
value to a vector-wise value"): the absmax is taken per output column, and the result is what
the library's int8 entry points consume (`wgpt_matmul_bias_i8`, `<stem>.weight.q` +
`<stem>.weight.scale` of `wgpt_model_set_tensor`):

    q[k, n]      = Math.round(W[k, n] / absmax[n] * 127) & 0xff      (JS numbers: float64)
    words[k, j]  = q[k, 4j] | q[k, 4j+1] << 8 | q[k, 4j+2] << 16 | q[k, 4j+3] << 24
    scale[n]     = absmax[n]                                          (float32, exact)

`Math.round` rounds halves toward +infinity (Math.round(-0.5) is -0, Math.round(2.5) is 3);
`NaN & 0xff` is 0, which is what an all-zero column (absmax 0) quantises to.

`dequantizeMatrix` is other/int8-gemm.js:48-62 (float64 arithmetic, one rounding when the
value is stored into the Float32Array), again with the column's absmax. The kernels instead
compute `float(q) / 127.0f * scale[n]` in fp32 (the shader, int8-gemm.js:126-132), which can
differ from this by one ulp; `wgpt_dequant_i8` gives that one.
"""
import numpy as np

LINEAR_STEMS = ("attn.c_attn", "attn.c_proj", "mlp.c_fc", "mlp.c_proj")


def _js_round(x):
    """Math.round on float64: the integer r with r <= x + 0.5 < r + 1, computed without forming x + 0.5
    (which rounds up for the double just below 0.5)."""
    r = np.floor(x)
    return r + ((x - r) >= 0.5)


def absmax_columns(W):
    """max_k |W[k, n]| in float64, as the reference's running Math.max over Math.abs (int8-gemm.js:29-33)."""
    W = np.asarray(W)
    if W.ndim != 2:
        raise ValueError("quantizeMatrix: a [K, N] matrix is required")
    return np.abs(W.astype(np.float64)).max(axis=0) if W.shape[0] else np.zeros(W.shape[1])


def quantizeMatrix(W, absmax=None):
    """(words int32 [K, N/4], scale float32 [N]) of an fp32 weight W[K, N] ([in, out], row-major).
    `absmax` overrides the per-column maxima (a scalar gives the reference's single global value)."""
    W = np.ascontiguousarray(W, dtype=np.float32)
    if W.ndim != 2:
        raise ValueError("quantizeMatrix: a [K, N] matrix is required")
    K, N = W.shape
    if N % 4 != 0:
        raise ValueError("Cols must be divisible by 4.")
    am = absmax_columns(W) if absmax is None else np.broadcast_to(np.asarray(absmax, np.float64), (N,))
    words = np.empty((K, N // 4), np.uint32)
    rows = max(1, (1 << 22) // max(N, 1))           # float64 temporaries of a few tens of MB
    with np.errstate(divide="ignore", invalid="ignore"):
        for k0 in range(0, K, rows):
            x = (W[k0:k0 + rows].astype(np.float64) / am) * 127.0
            q = _js_round(x)
            q = np.where(np.isfinite(q), q, 0.0)     # NaN & 0xff and Infinity & 0xff are 0 in JS
            b = (q.astype(np.int64) & 0xFF).astype(np.uint32).reshape(-1, N // 4, 4)
            words[k0:k0 + rows] = b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16) | (b[..., 3] << 24)
    return words.view(np.int32), am.astype(np.float32)


def unpack_bytes(words, N=None):
    """The signed bytes [K, N] of packed words [K, N/4] (`(w << 24) >> 24` ... `w >> 24`)."""
    words = np.ascontiguousarray(words, dtype=np.int32)
    K = words.shape[0]
    b = words.view(np.int8).reshape(K, -1)
    return b if N is None else b[:, :N]


def dequantizeMatrix(words, scale, K=None, N=None):
    """float32 [K, N] of other/int8-gemm.js:48-62: `(byte / 127.0) * absmax` in float64, rounded once."""
    b = unpack_bytes(words).astype(np.float64)
    s = np.asarray(scale, np.float64).reshape(-1)
    if K is not None and (b.shape[0] != K or (N is not None and b.shape[1] != N)):
        raise ValueError("dequantizeMatrix: packed words do not have the stated shape")
    return ((b / 127.0) * s).astype(np.float32)


def quantize_tensors(tensors):
    """A weight directory {name: array} with every fp32 linear weight `<stem>.weight` replaced by
    `<stem>.weight.q` and `<stem>.weight.scale`; everything else (embeddings, biases, LayerNorm) is kept."""
    out = {}
    for name, a in tensors.items():
        if name.startswith("transformer.h.") and name.endswith(".weight") and name.split(".", 3)[3][:-7] in LINEAR_STEMS:
            q, s = quantizeMatrix(a)
            out[name + ".q"], out[name + ".scale"] = q, s
        else:
            out[name] = a
    return out
