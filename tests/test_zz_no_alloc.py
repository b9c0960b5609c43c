"""wgpt_matmul_bias_noalloc: the matrix-vector product for callers that cannot allocate device memory. Its partial
sums live in a fixed array inside the library's code object; the result must be that of wgpt_matmul_bias, bit for
bit (same kernels, same order of additions), and within the parity bar of the oracle. Two calls in a row share the
array, the second with a smaller input: nothing of the first call may leak into it."""
import numpy as np
import pytest

from oracle import ref
from webgpt_amd import WgptError, _lib, blocks

from helpers import close, worst

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(123)


def both(M, N, K, with_bias=True):
    A = (RNG.standard_normal((M, K))).astype(np.float32)
    W = (RNG.standard_normal((K, N)) * 0.05).astype(np.float32)
    b = (RNG.standard_normal(N)).astype(np.float32) if with_bias else None
    ab, wb = blocks.init_tensor(A, [M, K]), blocks.init_tensor(W, [K, N])
    bb = blocks.init_tensor(b, [N]) if with_bias else None
    c0, c1 = blocks.Buffer([M, N]), blocks.Buffer([M, N])
    c1.upload(np.full(M * N, np.nan, np.float32))
    _lib.call("wgpt_matmul_bias", M, N, K, ab.handle, wb.handle, bb.handle if bb else 0, c0.handle)
    _lib.call("wgpt_matmul_bias_noalloc", M, N, K, ab.handle, wb.handle, bb.handle if bb else 0, c1.handle)
    got0, got1 = c0.download().reshape(M, N), c1.download().reshape(M, N)
    for x in (ab, wb, bb, c0, c1):
        if x is not None:
            x.destroy()
    return got0, got1, ref.matmul_bias(A, W, b)


def test_no_alloc_matmul_two_calls_in_a_row(device):
    print("wgpt_matmul_bias_noalloc: 4x3072x768 then 1x776x260", flush=True)
    for M, N, K, bias in ((4, 3072, 768, True), (1, 776, 260, False)):       # the second smaller, ragged in N and K
        want_lib, got, want = both(M, N, K, bias)
        assert np.array_equal(got.view(np.uint32), want_lib.view(np.uint32)), (M, N, K)
        assert close(got, want), (M, N, K, worst(got, want))


def test_no_alloc_matmul_limits(device):
    a = blocks.Buffer([8])
    with pytest.raises(WgptError, match="exceeds the 4 rows"):
        _lib.call("wgpt_matmul_bias_noalloc", 5, 8, 8, a.handle, a.handle, 0, a.handle)
    with pytest.raises(WgptError, match="exceed the fixed workspace"):
        _lib.call("wgpt_matmul_bias_noalloc", 4, 8192, 4096, a.handle, a.handle, 0, a.handle)   # 64 * 4 * 8192 = 2 Mi floats
    with pytest.raises(WgptError, match="divisible by 16"):
        _lib.call("wgpt_matmul_bias_noalloc", 1, 12, 8, a.handle, a.handle, 0, a.handle)
    a.destroy()
