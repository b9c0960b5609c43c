"""Token selection of GPT.generate (model.js:81-85; globals.js:47-74) on the device:
selectTopK + cpuSoftmax + sampleFromDistribution, with the uniform draw supplied."""
import ctypes as C

import numpy as np
import pytest
from scipy.special import softmax

from webgpt_amd import synth

from helpers import make_model, oracle_weights, small_cfg


def brute(logits, top_k, temperature, u):
    """Independent restatement: numpy stable argsort of the negated logits, scipy softmax."""
    x = np.asarray(logits, np.float32)
    order = np.argsort(-x.astype(np.float64), kind="stable")[:top_k]
    p = softmax(x[order].astype(np.float64) / temperature)
    cum = np.cumsum(p)
    hit = np.nonzero(u < cum)[0]
    pick = int(hit[0]) if hit.size else len(order) - 1
    return int(order[pick]), order.astype(np.int32), p


def cases():
    rng = np.random.default_rng(11)
    out = []
    for V, k, T in ((1, 1, 1.0), (5, 3, 1.0), (5, 9, 0.5), (65, 2, 1.0), (1000, 40, 0.7), (50257, 1, 1.0), (50257, 3, 1.0),
                    (50257, 50, 1.3), (4099, 1024, 2.0), (70001, 5, 1.0)):
        x = (rng.standard_normal(V) * 3).astype(np.float32)
        if V > 4:
            x[rng.integers(0, V, 6)] = x.max() + 1.0      # ties at the top: the lowest index must come first
            x[rng.integers(0, V, 6)] = x[0]
        for u in (0.0, 0.37, 0.93, 1.0 - 2.0 ** -53):
            out.append((x, k, T, u))
    return out


def test_oracle_selection_against_numpy_and_scipy():
    from oracle import ref
    for x, k, T, u in cases():
        want_id, want_ids, want_p = brute(x, k, T, u)
        got_id, ids, p = ref.sample_topk(x, k, T, u)
        assert np.array_equal(ids, want_ids)
        assert np.allclose(p, want_p, rtol=1e-13, atol=0)
        assert got_id == want_id
    # closed forms: equal logits -> uniform probabilities, draw u picks floor(u * k);
    # the stable order keeps ascending indices (globals.js:66-74)
    x = np.full(8, 0.25, np.float32)
    for u, want in ((0.0, 0), (0.26, 2), (0.99, 7)):
        got_id, ids, p = ref.sample_topk(x, 8, 1.0, u)
        assert list(ids) == list(range(8)) and np.allclose(p, 0.125) and got_id == want
    # two logits ln(3) apart at temperature 1: probabilities 3/4 and 1/4
    got_id, ids, p = ref.sample_topk(np.array([0.0, np.log(3.0)], np.float32), 2, 1.0, 0.76)
    assert list(ids) == [1, 0] and np.allclose(p, [0.75, 0.25], rtol=1e-7) and got_id == 0
    # temperature divides inside the exponent: T = 2 turns 3:1 into sqrt(3):1
    _, _, p = ref.sample_topk(np.array([0.0, np.log(3.0)], np.float32), 2, 2.0, 0.0)
    assert np.allclose(p[0] / p[1], np.sqrt(3.0), rtol=1e-7)


@pytest.mark.gpu
def test_device_selection_matches_oracle(device):
    from oracle import ref
    from webgpt_amd import _lib, blocks
    for x, k, T, u in cases():
        buf = blocks.init_tensor(x, [x.size])
        kk = min(k, x.size)
        cid = C.c_int32(-1)
        ids = np.empty(kk, np.int32)
        p = np.empty(kk, np.float64)
        _lib.call("wgpt_sample_topk", x.size, k, float(T), float(u), buf.handle, C.byref(cid),
                  ids.ctypes.data_as(C.POINTER(C.c_int32)), p.ctypes.data_as(C.POINTER(C.c_double)))
        want_id, want_ids, want_p = ref.sample_topk(x, k, T, u)
        assert np.array_equal(ids, want_ids), (x.size, k)          # index work: exact
        assert np.allclose(p, want_p, rtol=1e-12, atol=0)          # float64 exp: a few ulp between libraries
        assert cid.value == want_id
        buf.destroy()


@pytest.mark.gpu
def test_device_selection_rejects_bad_arguments(device):
    from webgpt_amd import _lib, blocks
    buf = blocks.init_tensor(np.zeros(8, np.float32), [8])
    cid = C.c_int32(0)
    for args, msg in (((8, 0, 1.0, 0.5), "top_k"), ((8, 2, 0.0, 0.5), "temperature"), ((8, 2, 1.0, 1.0), "u must be"),
                      ((9, 2, 1.0, 0.5), "wgpt_sample_topk")):
        with pytest.raises(_lib.WgptError, match=msg):
            _lib.call("wgpt_sample_topk", args[0], args[1], args[2], args[3], buf.handle, C.byref(cid), None, None)
    buf.destroy()


@pytest.mark.gpu
@pytest.mark.parametrize("mode,top_k", [(0, 5), (1, 2), (1, 5), (1, 8), (1, 9)])
def test_decode_sample_follows_the_reference_loop(device, mode, top_k):
    """wgpt_decode_sample == per token: logits of the window (oracle), then model.js:81-85.
    Mode 1 selects and samples inside the persistent kernel up to top_k = 8 and per token with the
    selection kernel above that."""
    from oracle import ref
    from webgpt_amd.model import GPT
    cfg = small_cfg(n_layer=2, n_head=6, n_embd=384, n_ctx=48, vocab_size=300)
    tensors = make_model(cfg, 21)
    params = synth.model_params(cfg)
    gpt = GPT(None, "char", tensors=tensors, params=params)
    gpt.initialize()
    try:
        try:
            gpt.set_decode_mode(mode)
        except _lib_error() as e:
            pytest.skip(str(e))
        prompt = [int(t) for t in synth.tokens(21, "prompt", 10, cfg["vocab_size"])]
        rng = np.random.default_rng(5)
        u = rng.random(12)
        T = 0.8
        lg = gpt.prefill(prompt)
        first, _, _ = ref.sample_topk(lg, top_k, T, 0.5)
        got = gpt.decode_sample(first, len(u), top_k, T, u)
        w = oracle_weights(tensors, cfg)
        hist = prompt + [first]
        for i, ui in enumerate(u):
            want_logits = ref.forward(params, w, np.array(hist, np.int32))
            want, ids, p = ref.sample_topk(want_logits, top_k, T, ui)
            # identical unless the draw sits within the parity tolerance of a boundary of the distribution
            cum = np.cumsum(p)
            near = np.min(np.abs(cum - ui)) < 1e-3 or (len(ids) == top_k and
                   np.sort(want_logits)[-top_k] - np.sort(want_logits)[-top_k - 1] < 1e-3)
            assert int(got[i]) == want or near, (i, int(got[i]), want)
            hist.append(int(got[i]))
    finally:
        gpt.unloadBuffers()


@pytest.mark.gpu
@pytest.mark.parametrize("top_k", [1, 3, 12])
def test_generate_in_bursts_yields_the_tokens_of_a_call_per_token(device, monkeypatch, top_k):
    """GPT.generate makes up to `burst` tokens per call once the window is cached, each with the draw the
    reference's loop (model.js:53-102) would have made for it: same ids as one call per token, also across
    the end of the context (sliding window) and when max_new_tokens is no multiple of the burst."""
    import random
    import time
    from webgpt_amd.model import GPT
    cfg = small_cfg(n_layer=2, n_head=6, n_embd=384, n_ctx=40, vocab_size=300)
    tensors = make_model(cfg, 22)
    gpt = GPT(None, "char", tensors=tensors, params=synth.model_params(cfg))
    gpt.initialize()
    try:
        prompt = [int(t) for t in synth.tokens(22, "prompt", 9, cfg["vocab_size"])]
        out, ms = {}, {}
        for burst in (1, 8, 5):
            gpt.burst = burst
            random.seed(1234)
            gpt._history = []
            t0 = time.perf_counter()
            out[burst] = [int(t) for t in gpt.generate(prompt, 43, top_k, 0.9)]   # runs past the 40 positions of the context
            ms[burst] = (time.perf_counter() - t0) * 1000.0 / 43
        print("generate ms/token by burst", {b: round(v, 4) for b, v in ms.items()})
        assert len(out[1]) == 43
        assert out[8] == out[1] and out[5] == out[1]
    finally:
        gpt.unloadBuffers()


def _lib_error():
    from webgpt_amd import _lib
    return _lib.WgptError


@pytest.mark.gpu
def test_decode_sample_rejects_bad_arguments(device):
    from webgpt_amd import _lib
    from webgpt_amd.model import GPT
    cfg = small_cfg(n_ctx=8)
    gpt = GPT(None, "char", tensors=make_model(cfg, 1), params=synth.model_params(cfg))
    gpt.initialize()
    try:
        gpt.prefill([1, 2, 3])
        for args, msg in (((4, 1, 0, 1.0, [0.5]), "top_k"), ((4, 1, 2000, 1.0, [0.5]), "top_k"), ((4, 1, 2, 0.0, [0.5]), "temperature"),
                          ((4, 1, 2, 1.0, [1.0]), r"u\[0\]"), ((cfg["vocab_size"], 1, 2, 1.0, [0.5]), "outside"),
                          ((4, 6, 2, 1.0, [0.5] * 6), "exceed")):
            with pytest.raises(_lib.WgptError, match=msg):
                gpt.decode_sample(*args)
        with pytest.raises(ValueError, match="one uniform draw per step"):
            gpt.decode_sample(4, 2, 2, 1.0, [0.5])
        assert len(gpt.decode_sample(4, 2, 3, 1.0, [0.1, 0.9])) == 2     # still usable afterwards
    finally:
        gpt.unloadBuffers()
