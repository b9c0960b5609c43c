"""Pins the CPU oracle (oracle/wgpt_oracle.c) without the reference runtime.

The reference holds no golden vectors that exist in this tree (its validation JSONs
are Git-LFS stubs), so every kernel restatement is checked against something it was
not derived from: float64 numpy brute force, torch CPU library routines, closed
forms and invariants, and the closed-form input of other/test.js:370-388.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import ref

RNG = np.random.default_rng(1234)


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


# ---------------- K1 fastMatMul ----------------

@pytest.mark.parametrize("M,N,K", [(1, 8, 4), (1, 64, 48), (3, 24, 20), (4, 72, 64), (5, 8, 12), (17, 264, 100),
                                   (64, 768, 384), (2, 520, 8)])
def test_matmul_vs_float64(M, N, K):
    A, B, b = rnd(M, K), rnd(K, N), rnd(N)
    got = ref.matmul_bias(A, B, b)
    want = A.astype(np.float64) @ B.astype(np.float64) + b
    # forward error bound of a length-K recursive sum in fp32
    bound = (K + 2) * 2.0 ** -24 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64) + np.abs(b)) + 1e-30
    assert np.all(np.abs(got - want) <= bound)


def test_matmul_exact_cases():
    # identity weights: the only non-zero product is a*1, every other term adds +0
    A, b = rnd(6, 32), rnd(32)
    assert np.array_equal(ref.matmul_bias(A, np.eye(32, dtype=np.float32), b), A + b)
    # one-hot rows pick rows of B exactly
    B = rnd(16, 40)
    A = np.zeros((3, 16), np.float32)
    A[0, 5] = A[1, 0] = A[2, 15] = 1.0
    assert np.array_equal(ref.matmul_bias(A, B, None), B[[5, 0, 15]])
    # small integers: exact in fp32, so any order or index mistake shows
    A = RNG.integers(-8, 9, (7, 12)).astype(np.float32)
    B = RNG.integers(-8, 9, (12, 16)).astype(np.float32)
    b = RNG.integers(-8, 9, 16).astype(np.float32)
    assert np.array_equal(ref.matmul_bias(A, B, b), A @ B + b)


def test_matmul_order_is_ascending_k_then_bias():
    # A sum whose value depends on the order: 1e8 + 1 - 1e8 in fp32.
    A = np.array([[1.0, 1.0, 1.0]], np.float32)
    B = np.zeros((3, 8), np.float32)
    B[:, 0] = [1e8, 1.0, -1e8]      # ((0+1e8)+1)-1e8 = 0 in fp32
    B[:, 1] = [1.0, 1e8, -1e8]      # ((0+1)+1e8)-1e8 = 0
    B[:, 2] = [1e8, -1e8, 1.0]      # = 1
    bias = np.zeros(8, np.float32)
    bias[3] = 1.0
    B[:, 3] = [1e8, -1e8, 0.0]      # bias added last: 0 + 1 = 1
    out = ref.matmul_bias(A, B, bias)[0]
    assert out[0] == 0.0 and out[1] == 0.0 and out[2] == 1.0 and out[3] == 1.0


# ---------------- K2 residual ----------------

def test_residual_exact():
    a, b = rnd(5, 16), rnd(5, 16)
    assert np.array_equal(ref.residual(a, b), a + b)


# ---------------- K3/K4 layer norm ----------------

@pytest.mark.parametrize("M,N", [(1, 64), (3, 384), (5, 768), (2, 1600), (2, 4100), (4, 32)])
def test_layernorm_vs_torch_and_float64(M, N):
    x, g, b = rnd(M, N, scale=3.0) + 0.7, rnd(N), rnd(N)
    got = ref.layernorm(x, g, b)
    want_t = F.layer_norm(torch.from_numpy(x), (N,), torch.from_numpy(g), torch.from_numpy(b), eps=1e-5).numpy()
    x64 = x.astype(np.float64)
    mu = x64.mean(1, keepdims=True)
    var = ((x64 - mu) ** 2).mean(1, keepdims=True)
    want = g * ((x64 - mu) / np.sqrt(var + 1e-5)) + b
    assert np.allclose(got, want, rtol=1e-5, atol=2e-6)
    assert np.allclose(got, want_t, rtol=1e-5, atol=4e-6)


def test_layernorm_stats_and_invariants():
    x = rnd(4, 768, scale=2.0) + 5.0
    st = ref.layernorm_stats(x)
    x64 = x.astype(np.float64)
    assert np.allclose(st[:, 0], x64.mean(1), rtol=1e-6)
    assert np.allclose(st[:, 1], np.sqrt(x64.var(1) + 1e-5), rtol=1e-5)   # biased variance, eps inside the sqrt
    y = ref.layernorm(x, np.ones(768, np.float32), np.zeros(768, np.float32))
    assert np.allclose(y.mean(1), 0, atol=1e-5) and np.allclose(y.var(1), 1, atol=1e-3)
    # a constant row has zero variance: output is beta, stdev is sqrt(1e-5)
    c = np.full((1, 64), 3.25, np.float32)
    beta = rnd(64)
    assert np.array_equal(ref.layernorm(c, rnd(64), beta), beta[None, :])
    assert ref.layernorm_stats(c)[0, 1] == np.sqrt(np.float32(1e-5))


# ---------------- K5 softmax ----------------

@pytest.mark.parametrize("M,N", [(1, 1), (3, 7), (4, 64), (2, 65), (6, 1000), (2, 5000)])
def test_softmax_vs_float64(M, N):
    x = rnd(M, N, scale=4.0)
    got = ref.softmax(x)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(1, keepdims=True))
    assert np.allclose(got, e / e.sum(1, keepdims=True), rtol=2e-6, atol=1e-9)
    assert np.allclose(got.sum(1), 1, atol=1e-5)


def test_softmax_masked_row_and_shift():
    x = np.full((1, 40), -1e9, np.float32)
    x[0, 17] = 0.3
    out = ref.softmax(x)
    assert out[0, 17] == 1.0 and np.count_nonzero(out) == 1       # exp(-1e9 - 0.3) underflows to exactly 0
    y = rnd(2, 33)
    assert np.allclose(ref.softmax(y), ref.softmax(y + np.float32(8.0)), rtol=1e-5)


# ---------------- K6 GELU ----------------

def test_gelu_vs_torch_and_thresholds():
    x = np.concatenate([rnd(1000, scale=3.0), np.linspace(-9.99, 9.99, 400).astype(np.float32)]).reshape(1, -1)
    x = x[:, : x.shape[1] // 4 * 4]
    got = ref.gelu(x)
    want = F.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    edge = np.array([[-10.5, -10.0, 10.0, 10.5, -1e30, 1e30, 0.0, -0.0]], np.float32)
    out = ref.gelu(edge)[0]
    assert out[0] == 0.0 and out[3] == np.float32(10.5) and out[4] == 0.0 and out[5] == np.float32(1e30)
    assert out[6] == 0.0
    # x*Phi(x) + x*Phi(-x) = x for the tanh form: gelu(x) - gelu(-x) = x
    z = rnd(1, 64, scale=2.0)
    assert np.allclose(ref.gelu(z) - ref.gelu(-z), z, atol=1e-6)


# ---------------- embed / de-embed ----------------

def test_embed_and_deembed():
    V, d, T = 65, 32, 9
    wte, wpe = rnd(V, d), rnd(16, d)
    idx = RNG.integers(0, V, T).astype(np.int32)
    assert np.array_equal(ref.embed(idx, wte, wpe), wte[idx] + wpe[:T])
    x = rnd(T, d)
    got = ref.deembed(x, wte)
    want = wte.astype(np.float64) @ x[-1].astype(np.float64)        # last row only, tied weights, no bias
    assert got.shape == (V,) and np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # the reference multiplies by the transposed table: same numbers as K1 on wte^T
    assert np.array_equal(got, ref.matmul_bias(x[-1:], np.ascontiguousarray(wte.T), None)[0])


# ---------------- attention pieces ----------------

def test_format_q_is_the_head_split_permutation():
    T, H, hs = 5, 3, 8
    Q = rnd(T, H * hs)
    assert np.array_equal(ref.format_q(Q, hs), Q.reshape(T, H, hs).transpose(1, 0, 2))


def test_attn_weights_brute_force_and_mask():
    T, H, hs = 6, 2, 8
    Q, Km = rnd(T, H * hs), rnd(T, H * hs)
    scale = np.float32(1 / math.sqrt(hs))
    S = ref.attn_weights(ref.format_q(Q, hs), Km, scale).reshape(H, T, T)
    for h in range(H):
        for i in range(T):
            for j in range(T):
                if j > i:
                    assert S[h, i, j] == np.float32(-1e9)
                else:
                    want = float(np.dot(Q[i, h * hs:(h + 1) * hs].astype(np.float64), Km[j, h * hs:(h + 1) * hs])) / math.sqrt(hs)
                    assert abs(S[h, i, j] - want) < 1e-5
    assert np.float32(1 / math.sqrt(64)) == np.float32(0.125)


def test_attn_values_known_answer_of_reference_test_js():
    # other/test.js:370-388: T=15, d=128, H=4; P[h*T+i, j] = h+1 for j <= i else 0; V[j, c] = c // hs + 1.
    # Closed form: O[i, c] = (i + 1) * (c // hs + 1) ** 2.
    T, d, H = 15, 128, 4
    hs = d // H
    P = np.zeros((H * T, T), np.float32)
    for y in range(H * T):
        for x in range(T):
            P[y, x] = y // T + 1 if x <= y % T else 0
    V = np.tile((np.arange(d) // hs + 1).astype(np.float32), (T, 1))
    O = ref.attn_values(P, V, hs)
    want = np.array([[(i + 1) * (c // hs + 1) ** 2 for c in range(d)] for i in range(T)], np.float32)
    assert np.array_equal(O, want)


@pytest.mark.parametrize("T,H,hs", [(1, 2, 8), (7, 3, 16), (33, 4, 64)])
def test_attention_block_vs_torch_float64(T, H, hs):
    d = H * hs
    x = rnd(T, d)
    W = [rnd(d, d, scale=0.5 / math.sqrt(d)) for _ in range(4)]
    b = [rnd(d, scale=0.1) for _ in range(4)]
    got, Kc, Vc = ref.attention(x, W[0], b[0], W[1], b[1], W[2], b[2], W[3], b[3], H, return_kv=True)
    t = lambda a: torch.from_numpy(a).double()
    q, k, v = (t(x) @ t(W[i]) + t(b[i]) for i in range(3))
    split = lambda a: a.reshape(T, H, hs).transpose(0, 1)
    o = F.scaled_dot_product_attention(split(q), split(k), split(v), is_causal=True)
    want = (o.transpose(0, 1).reshape(T, d) @ t(W[3]) + t(b[3])).numpy()
    assert np.allclose(got, want, rtol=1e-4, atol=1e-5)
    assert np.allclose(Kc, k.numpy(), atol=1e-5) and np.allclose(Vc, v.numpy(), atol=1e-5)


# ---------------- int8 weight-only ----------------

def test_int8_dequant_exhaustive_bit_exact():
    # every byte value x a set of scales, against IEEE fp32 arithmetic done by numpy:
    # f32(b) / 127.0f rounded, then * scale rounded (other/int8-gemm.js:127-130)
    scales = np.array([1e-3, 9.999e-3, 0.0123456, 1.0, 3.1415927, 1e-8, 127.0, 5.5e-3], np.float32)
    bytes_ = np.arange(-128, 128, dtype=np.int64)
    K, N = 256, 8
    q = np.repeat(bytes_[:, None], N, axis=1)
    packed = ((q.reshape(K, N // 4, 4) & 0xFF).astype(np.uint32) << np.array([0, 8, 16, 24], np.uint32)).sum(-1).astype(np.uint32).view(np.int32)
    got = ref.dequant_i8(packed, scales, N)
    want = (q.astype(np.float32) / np.float32(127.0)) * scales[None, :]
    assert want.dtype == np.float32 and np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_int8_sign_extension_per_byte_lane():
    # 0x80 in each lane is -128 there and 0 elsewhere; 0x7f is +127
    for e in range(4):
        word = np.array([[np.uint32(0x80 << (8 * e))]], np.uint32).view(np.int32)
        out = ref.dequant_i8(word, np.full(4, 127.0, np.float32), 4)[0]
        want = np.zeros(4, np.float32)
        want[e] = -128.0
        assert np.array_equal(out, want)
        word = np.array([[np.uint32(0x7F << (8 * e))]], np.uint32).view(np.int32)
        assert ref.dequant_i8(word, np.full(4, 127.0, np.float32), 4)[0][e] == 127.0


def test_int8_quantize_matches_js_semantics_and_round_trip():
    w = rnd(64, scale=0.1)
    w[5] = 0.0
    packed, absmax = ref.quantize_global(w)
    amax = float(np.abs(w).max())
    assert absmax == np.float32(amax)
    by = packed.view(np.uint8).reshape(-1)
    for i, v in enumerate(w):
        q = math.floor((float(v) / amax) * 127 + 0.5)        # Math.round: half toward +infinity
        assert by[i] == (q & 0xFF)
    # JS dequantizeMatrix is double arithmetic with one rounding
    dq = ref.dequantize_js(packed, absmax, 64)
    sb = by.view(np.int8).astype(np.float64)
    assert np.array_equal(dq, ((sb / 127.0) * float(absmax)).astype(np.float32))
    assert np.max(np.abs(dq - w)) <= amax / 127 * 0.5001
    # Math.round(-0.5) is -0 -> byte 0; Math.round(0.5) is 1; Math.round(-1.5) is -1
    probe = np.array([-0.5 / 127, 0.5 / 127, -1.5 / 127, 1.0], np.float64).astype(np.float32)
    pk, am = ref.quantize_global(probe)
    assert am == 1.0
    got = pk.view(np.int8)[:4]
    want = [math.floor(float(v) * 127 + 0.5) for v in probe]
    assert list(got) == want


def test_int8_matmul_equals_fp32_matmul_on_dequantised_weights():
    M, K, N = 3, 40, 24
    A = rnd(M, K)
    q = RNG.integers(-127, 128, (K, N))
    packed = ((q.reshape(K, N // 4, 4) & 0xFF).astype(np.uint32) << np.array([0, 8, 16, 24], np.uint32)).sum(-1).astype(np.uint32).view(np.int32)
    scale = RNG.uniform(1e-3, 1e-2, N).astype(np.float32)
    bias = rnd(N)
    W = ref.dequant_i8(packed, scale, N)
    assert np.array_equal(ref.matmul_i8(A, packed, scale, bias), ref.matmul_bias(A, W, bias))
    assert np.array_equal(ref.matmul_i8(A, packed, scale, None), ref.matmul_bias(A, W, None))
