"""Parity of every instruction block, called through the C ABI (via the block
mirror of webgpt_amd/blocks.py), against the CPU oracle on the same seeded inputs.
fp32 bar: |got - want| <= 1e-5 + 1e-4 |want|; copies, gathers and the int8
dequantisation are bit-exact."""
import math

import numpy as np
import pytest

from oracle import ref
from webgpt_amd import WgptError, blocks
from webgpt_amd.blocks import (AttentionBlock, DeEmbedBlock, EmbedBlock, FastMatMulBlock, GeluBlock, LayerNormBlock,
                               ResidualBlock, SoftmaxBlock, init_tensor, run_passes)

from helpers import close, pack_words, worst

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(99)


def rnd(*shape, scale=1.0):
    return (RNG.standard_normal(shape) * scale).astype(np.float32)


def run(inst, shape):
    run_passes(inst["passes"])
    out = inst["resultBuffer"].download().reshape(shape)
    blocks.clearOperationCache()
    return out


@pytest.mark.parametrize("M,N,K", [(1, 8, 4), (1, 768, 768), (1, 2304, 768), (1, 768, 3072), (1, 72, 100), (2, 64, 64),
                                   (3, 1600, 1600), (4, 384, 1536), (5, 8, 12), (7, 200, 36), (16, 768, 768),
                                   (128, 2304, 768), (65, 136, 260), (200, 768, 3072), (2048, 4096, 64), (2050, 4104, 40),
                                   # short prompts: K split over the waves of a workgroup (32x32 and 16x16 blocks, ragged M,
                                   # K steps that do not divide by the eight waves)
                                   (17, 32, 128), (100, 1600, 1600), (250, 96, 3200), (33, 6400, 1600), (256, 384, 384), (31, 64, 144),
                                   # the two-group kernel: K split four ways, one tile per compute unit, ragged M and N
                                   # with an odd number of K steps, and the same shape with a ragged K (other kernel)
                                   (512, 1024, 1024), (512, 4096, 1024), (950, 2056, 96), (950, 2056, 100)])
def test_fast_matmul(device, M, N, K):
    A, W, b = rnd(M, K), rnd(K, N, scale=0.05), rnd(N)
    inst = FastMatMulBlock.newInstance(M, N, K, init_tensor(A, [M, K]), init_tensor(W, [K, N]), init_tensor(b, [N]))
    got = run(inst, (M, N))
    want = ref.matmul_bias(A, W, b)
    assert close(got, want), worst(got, want)


def _dispatch_edge_shapes():
    """Seeded shapes around the tile counts at which the matmul changes kernel or K split (64x128 tiles in whole
    rounds of 256 workgroups, 64x64 tiles otherwise), with ragged M, N and K among them."""
    rng = np.random.default_rng(20240607)
    shapes = []
    for tiles in (63, 64, 65, 127, 128, 218, 255, 256, 257, 435, 512, 513, 1023, 1024, 1025):
        mt = int(rng.integers(2, 17))                      # rows of 64
        nt = max(1, tiles // mt)                           # columns of 128
        M = 64 * mt - int(rng.integers(0, 40))
        N = 128 * nt - 8 * int(rng.integers(0, 8))
        K = int(rng.choice([32, 96, 100, 128, 256, 260, 512, 1024]))
        shapes.append((max(M, 5), max(N, 8), K))
    return shapes


@pytest.mark.parametrize("M,N,K", [(128, 2304, 768), (64, 1536, 640), (128, 768, 672), (100, 768, 576), (448, 512, 768),
                                   (449, 512, 768), (128, 1600, 6400), (33, 4800, 1600)])
def test_fast_matmul_with_few_rows_and_odd_slice_counts(device, M, N, K):
    # up to 448 rows the K range is cut into any number of slices that leaves whole steps of 32 (here 3, 5, 7, 6, ...),
    # not only powers of two; 449 rows fall back to doubling. (Weights scaled with K: near a zero of the output the
    # rounding of 6400 fp32 additions, in whatever order, is otherwise larger than the absolute tolerance.)
    A, W, b = rnd(M, K), rnd(K, N, scale=0.05 * min(1.0, 1024.0 / K)), rnd(N)
    inst = FastMatMulBlock.newInstance(M, N, K, init_tensor(A, [M, K]), init_tensor(W, [K, N]), init_tensor(b, [N]))
    got = run(inst, (M, N))
    want = ref.matmul_bias(A, W, b)
    assert close(got, want), worst(got, want)


@pytest.mark.parametrize("M,N,K", _dispatch_edge_shapes())
def test_fast_matmul_around_kernel_choices(device, M, N, K):
    A, W, b = rnd(M, K), rnd(K, N, scale=0.05), rnd(N)
    inst = FastMatMulBlock.newInstance(M, N, K, init_tensor(A, [M, K]), init_tensor(W, [K, N]), init_tensor(b, [N]))
    got = run(inst, (M, N))
    want = ref.matmul_bias(A, W, b)
    assert close(got, want), worst(got, want)


def test_fast_matmul_exact_and_preconditions(device):
    A = RNG.integers(-8, 9, (3, 12)).astype(np.float32)
    W = RNG.integers(-8, 9, (12, 16)).astype(np.float32)
    b = RNG.integers(-8, 9, 16).astype(np.float32)
    bufs = init_tensor(A, [3, 12]), init_tensor(W, [12, 16]), init_tensor(b, [16])
    assert np.array_equal(run(FastMatMulBlock.newInstance(3, 16, 12, *bufs), (3, 16)), A @ W + b)
    with pytest.raises(ValueError, match="Cols must be divisible by 16."):
        FastMatMulBlock.newInstance(3, 12, 12, *bufs)
    # the library checks shapes against buffer sizes before any launch
    with pytest.raises(WgptError, match="buffer holds"):
        run_passes(FastMatMulBlock.newInstance(4, 16, 12, *bufs)["passes"])
    blocks.clearOperationCache()


@pytest.mark.parametrize("M,N", [(1, 4), (1, 768), (3, 384), (130, 1600)])
def test_residual_and_gelu(device, M, N):
    a, b = rnd(M, N, scale=3.0), rnd(M, N)
    got = run(ResidualBlock.newInstance(M, N, init_tensor(a, [M, N]), init_tensor(b, [M, N])), (M, N))
    assert np.array_equal(got, a + b)
    a[0, :4] = [-10.5, 10.5, -10.0, 10.0]
    got = run(GeluBlock.newInstance(M, N, init_tensor(a, [M, N])), (M, N))
    want = ref.gelu(a)
    assert close(got, want), worst(got, want)
    assert got[0, 0] == 0.0 and got[0, 1] == np.float32(10.5)


@pytest.mark.parametrize("M,N", [(1, 4), (1, 768), (5, 384), (64, 1600), (2, 4100), (3, 1024)])
def test_layernorm(device, M, N):
    x, g, b = rnd(M, N, scale=2.0) + 0.5, rnd(N), rnd(N)
    got = run(LayerNormBlock.newInstance(M, N, init_tensor(x, [M, N]), init_tensor(g, [N]), init_tensor(b, [N])), (M, N))
    want = ref.layernorm(x, g, b)
    assert close(got, want), worst(got, want)


@pytest.mark.parametrize("M,N", [(1, 1), (3, 7), (12, 64), (24, 129), (6, 1024), (2, 5000)])
def test_softmax(device, M, N):
    x = rnd(M, N, scale=3.0)
    if N > 2:
        x[0, 2:] = -1e9
    got = run(SoftmaxBlock.newInstance(M, N, init_tensor(x, [M, N])), (M, N))
    want = ref.softmax(x)
    assert close(got, want, atol=1e-7), worst(got, want, atol=1e-7)
    if N > 2:
        assert np.count_nonzero(got[0, 2:]) == 0


@pytest.mark.parametrize("M,N", [(1, 1), (3, 7), (24, 129), (65, 64)])
def test_softmax_transposed_store(device, M, N):
    # SoftmaxBlock.newInstance(rows, cols, in, transpose=true): out[i * M + row] (instructions.js:594)
    x = rnd(M, N, scale=3.0)
    inst = SoftmaxBlock.newInstance(M, N, init_tensor(x, [M, N]), True)
    assert tuple(inst["resultBuffer"].dims) == (N, M)
    got = run(inst, (N, M))
    plain = run(SoftmaxBlock.newInstance(M, N, init_tensor(x, [M, N])), (M, N))
    assert np.array_equal(got, plain.T)
    want = ref.softmax(x).T
    assert close(got, want, atol=1e-7), worst(got, want, atol=1e-7)


def test_chunked_vocabulary_buffers_as_the_reference_builds_them(device):
    """The reference holds the table as zero-padded chunks: [chunk, d] copies for the gather and host-transposed
    [d, chunk] copies for the de-embedding (model.js:298-364; 50257 rows -> two chunks of 25132). Both blocks accept
    such lists and give the single-table results bit for bit."""
    V, d, T, ctx, chunk = 50257, 768, 9, 32, 25132
    wte, wpe = rnd(V, d, scale=0.02), rnd(ctx, d, scale=0.02)
    padded = np.zeros((2 * chunk, d), np.float32)
    padded[:V] = wte
    gather = [init_tensor(padded[i * chunk:(i + 1) * chunk], [chunk, d]) for i in range(2)]
    transposed = [init_tensor(np.ascontiguousarray(padded[i * chunk:(i + 1) * chunk].T), [d, chunk]) for i in range(2)]
    idx = np.array([0, V - 1, 17, 17, 25131, 25132, 40000, 3, 50256], np.int32)
    wte_b, wpe_b = init_tensor(wte, [V, d]), init_tensor(wpe, [ctx, d])
    inst = EmbedBlock.newInstance(idx, T, d, chunk, gather, wpe_b, ResidualBlock)
    assert sum(p["flag"] == "copy" for p in inst["passes"]) == T + 1          # instructions.js:795-819
    got = run(inst, (T, d))
    assert np.array_equal(got, ref.embed(idx, wte, wpe))
    assert np.array_equal(got, run(EmbedBlock.newInstance(idx, T, d, V, [wte_b], wpe_b, ResidualBlock), (T, d)))
    x = rnd(T, d)
    x_b = init_tensor(x, [T, d])
    single = run(DeEmbedBlock.newInstance(d, V, V, T, V, x_b, [wte_b]), (V,))
    for _ in range(2):   # the second instance finds the chunks' row form already made
        inst = DeEmbedBlock.newInstance(d, V, 2 * chunk, T, chunk, x_b, transposed)
        assert [p["flag"] for p in inst["passes"]] == ["compute", "copy"] * 2      # instructions.js:858-882
        got = run(inst, (V,))
        assert np.array_equal(got, single)
    want = ref.deembed(x, wte)
    assert close(got, want), worst(got, want)
    with pytest.raises(ValueError, match="outside"):
        EmbedBlock.newInstance(np.array([2 * chunk], np.int32), 1, d, chunk, gather, wpe_b, ResidualBlock)
    for b in gather + transposed + [wte_b, wpe_b, x_b]:
        b.destroy()
    blocks.clearOperationCache()


def test_embed_and_deembed(device):
    V, d, T, ctx = 50257, 768, 9, 32
    wte, wpe = rnd(V, d, scale=0.02), rnd(ctx, d, scale=0.02)
    idx = np.array([0, V - 1, 17, 17, 25131, 25132, 40000, 3, 50256], np.int32)
    wte_b, wpe_b = init_tensor(wte, [V, d]), init_tensor(wpe, [ctx, d])
    got = run(EmbedBlock.newInstance(idx, T, d, V, [wte_b], wpe_b, ResidualBlock), (T, d))
    assert np.array_equal(got, ref.embed(idx, wte, wpe))
    x = rnd(T, d)
    got = run(DeEmbedBlock.newInstance(d, V, V, T, V, init_tensor(x, [T, d]), [wte_b]), (V,))
    want = ref.deembed(x, wte)
    assert close(got, want), worst(got, want)
    with pytest.raises(WgptError, match="outside"):
        run_passes(EmbedBlock.newInstance(np.array([V], np.int32), 1, d, V, [wte_b], wpe_b, ResidualBlock)["passes"])
    blocks.clearOperationCache()


def test_deembed_ragged_vocab(device):
    V, d, T = 65, 384, 3
    wte, x = rnd(V, d), rnd(T, d)
    got = run(DeEmbedBlock.newInstance(d, V, 68, T, 68, init_tensor(x, [T, d]), [init_tensor(wte, [V, d])]), (V,))
    want = ref.deembed(x, wte)
    assert close(got, want), worst(got, want)


@pytest.mark.parametrize("T,H,hs", [(1, 2, 8), (15, 4, 32), (64, 6, 64), (130, 12, 64), (5, 2, 4), (33, 25, 64), (20, 3, 64), (300, 2, 64)])
def test_attention(device, T, H, hs):
    d = H * hs
    x = rnd(T, d)
    W = [rnd(d, d, scale=0.5 / math.sqrt(d)) for _ in range(4)]
    b = [rnd(d, scale=0.1) for _ in range(4)]
    scale = 1 / math.sqrt(hs)
    bufs = [init_tensor(x, [T, d])]
    for i in range(4):
        bufs += [init_tensor(W[i], [d, d]), init_tensor(b[i], [d])]
    got = run(AttentionBlock.newFusedInstance(T, d, scale, H, hs, *bufs, FastMatMulBlock, SoftmaxBlock), (T, d))
    want = ref.attention(x, W[0], b[0], W[1], b[1], W[2], b[2], W[3], b[3], H)
    assert close(got, want), worst(got, want)


def test_attention_values_known_answer(device):
    # other/test.js:370-388 through the attention block: with Wq = Wk = 0 every score is 0, so the
    # softmax is uniform over j <= i: P = 1/(i+1). V = c // hs + 1 (via bv, Wv = 0), Wo = I:
    # O[i, c] = sum_{j<=i} (1/(i+1)) * (c // hs + 1) = c // hs + 1.
    T, d, H = 15, 128, 4
    hs = d // H
    z = np.zeros((d, d), np.float32)
    zb = np.zeros(d, np.float32)
    vrow = (np.arange(d) // hs + 1).astype(np.float32)
    bufs = [init_tensor(rnd(T, d), [T, d]), init_tensor(z, [d, d]), init_tensor(zb, [d]), init_tensor(z, [d, d]),
            init_tensor(zb, [d]), init_tensor(z, [d, d]), init_tensor(vrow, [d]),
            init_tensor(np.eye(d, dtype=np.float32), [d, d]), init_tensor(zb, [d])]
    got = run(AttentionBlock.newFusedInstance(T, d, 1 / math.sqrt(hs), H, hs, *bufs), (T, d))
    assert np.allclose(got, np.tile(vrow, (T, 1)), rtol=1e-6)


@pytest.mark.parametrize("M,N,K", [(1, 8, 4), (1, 1600, 1600), (1, 4800, 1600), (1, 1600, 6400), (3, 264, 100), (40, 136, 64), (130, 264, 100), (300, 4800, 1600), (512, 1600, 6400)])
def test_int8_matmul_and_bit_exact_dequant(device, M, N, K):
    A = rnd(M, K)
    q = RNG.integers(-127, 128, (K, N))
    q[0, :4] = [-128, 127, -1, 0]
    packed = pack_words(q)
    scale = RNG.uniform(1e-3, 1e-2, N).astype(np.float32)
    bias = rnd(N)
    pk, sc = init_tensor(packed, [K, N // 4]), init_tensor(scale, [N])
    # dequantised weights: bit-exact
    wbuf = blocks.Buffer([K, N])
    from webgpt_amd import _lib
    _lib.call("wgpt_dequant_i8", K, N, pk.handle, sc.handle, wbuf.handle)
    W = wbuf.download().reshape(K, N)
    wbuf.destroy()
    want_w = ref.dequant_i8(packed, scale, N)
    assert np.array_equal(W.view(np.uint32), want_w.view(np.uint32))
    inst = FastMatMulBlock.newInt8Instance(M, N, K, init_tensor(A, [M, K]), pk, sc, init_tensor(bias, [N]))
    got = run(inst, (M, N))
    want = ref.matmul_i8(A, packed, scale, bias)
    assert close(got, want), worst(got, want)


def test_int8_dequant_all_bytes(device):
    from webgpt_amd import _lib
    scales = np.array([1e-3, 9.999e-3, 0.0123456, 1.0, 3.1415927, 1e-8, 127.0, 5.5e-3], np.float32)
    q = np.repeat(np.arange(-128, 128)[:, None], 8, axis=1)
    packed = pack_words(q)
    pk, sc, out = init_tensor(packed, [256, 2]), init_tensor(scales, [8]), blocks.Buffer([256, 8])
    _lib.call("wgpt_dequant_i8", 256, 8, pk.handle, sc.handle, out.handle)
    got = out.download().reshape(256, 8)
    want = (q.astype(np.float32) / np.float32(127.0)) * scales[None, :]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), ref.dequant_i8(packed, scales, 8).view(np.uint32))
