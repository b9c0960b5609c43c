"""Parity of the whole-model path (wgpt_prefill / wgpt_decode / wgpt_decode_greedy,
called through the C ABI) against the CPU oracle's GPT.run restatement."""
import ctypes as C

import numpy as np
import pytest

from oracle import ref
from webgpt_amd import WgptError, _lib, synth
from webgpt_amd.model import GPT

from helpers import close, make_model, oracle_weights, small_cfg, worst

pytestmark = pytest.mark.gpu


def load(cfg, seed, flags=0, random_ln=True):
    tensors = make_model(cfg, seed, random_ln=random_ln)
    gpt = GPT(None, "char", tensors=tensors, params=synth.model_params(cfg), flags=flags)
    gpt.initialize()
    return gpt, tensors


def greedy_ok(got_logits, want_logits):
    """Greedy ids must agree unless the oracle's top-2 gap is inside the tolerance."""
    g, w = int(np.argmax(got_logits)), int(np.argmax(want_logits))
    if g == w:
        return True
    top2 = np.sort(want_logits)[-2:]
    return abs(float(top2[1] - top2[0])) <= 1e-5 + 1e-4 * abs(float(top2[1]))


@pytest.mark.parametrize("cfg,T", [(small_cfg(), 1), (small_cfg(), 9), (small_cfg(n_layer=3, n_head=4, n_embd=64, n_ctx=40, vocab_size=97), 40),
                                   (dict(synth.CONFIGS["toy"]), 64)])
def test_prefill_taps_and_logits(device, cfg, T):
    gpt, tensors = load(cfg, seed=11, flags=_lib.FLAG_TAPS)
    tokens = synth.tokens(5, "prompt", T, cfg["vocab_size"])
    want_logits, want_taps, want_kv = ref.forward(synth.model_params(cfg), oracle_weights(tensors, cfg), tokens,
                                                  want_taps=True, want_kv=True)
    logits = gpt.prefill(tokens)
    for i, name in enumerate(ref.tap_names(cfg["n_layer"])):
        got = gpt.tap(name, T)
        assert close(got, want_taps[i]), (name, worst(got, want_taps[i]))
    for i in range(cfg["n_layer"]):
        assert close(gpt.tap(f"kv{i}_k"), want_kv[i, 0]) and close(gpt.tap(f"kv{i}_v"), want_kv[i, 1])
    assert close(logits, want_logits), worst(logits, want_logits)
    assert greedy_ok(logits, want_logits)
    gpt.unloadBuffers()


@pytest.mark.parametrize("name,n_layer,T", [("toy", 6, 16), ("toy", 6, 33), ("toy", 3, 200), ("gpt2-117m", 2, 128), ("gpt2-1.5b", 1, 50)])
def test_short_prompt_prefill_against_oracle(device, name, n_layer, T):
    # prompts of 16..256 tokens run without taps (split-K products whose reduction pass applies the LayerNorm and
    # scatters the cache rows): logits and the cache rows they leave, then a decode step on top of them
    cfg = dict(synth.CONFIGS[name])
    cfg["n_layer"] = n_layer
    gpt, tensors = load(cfg, seed=23)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(9, "prompt", T + 1, cfg["vocab_size"])
    want, _, want_kv = ref.forward(p, w, tokens[:T], want_taps=True, want_kv=True)
    got = gpt.prefill(tokens[:T])
    assert close(got, want), worst(got, want)
    assert greedy_ok(got, want)
    for i in range(n_layer):
        assert close(gpt.tap(f"kv{i}_k"), want_kv[i, 0]), (i, worst(gpt.tap(f"kv{i}_k"), want_kv[i, 0]))
        assert close(gpt.tap(f"kv{i}_v"), want_kv[i, 1])
    got = gpt.decode(int(tokens[T]))
    want = ref.forward(p, w, tokens)
    assert close(got, want), worst(got, want)
    gpt.unloadBuffers()


def test_decode_equals_last_row_of_full_forward(device):
    # decode(t) with the KV cache must equal the reference's full-window recompute of tokens [0..t]
    cfg = dict(synth.CONFIGS["toy"])
    gpt, tensors = load(cfg, seed=7)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(3, "prompt", 40, cfg["vocab_size"])
    logits = gpt.run(tokens[:8])
    assert close(logits, ref.forward(p, w, tokens[:8]))
    for t in range(8, 40):
        logits = gpt.run(tokens[: t + 1])          # extends the window by one: served from the cache
        if t in (8, 9, 17, 31, 39):
            want = ref.forward(p, w, tokens[: t + 1])
            assert close(logits, want), (t, worst(logits, want))
            assert greedy_ok(logits, want)
    # a window that is not an extension recomputes from scratch
    other = synth.tokens(4, "prompt", 5, cfg["vocab_size"])
    assert close(gpt.run(other), ref.forward(p, w, other))
    gpt.unloadBuffers()


def test_greedy_generation_matches_oracle(device):
    cfg = dict(synth.CONFIGS["toy"])
    gpt, tensors = load(cfg, seed=1, random_ln=False)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    prompt = [int(t) for t in synth.make_prompt(cfg, 1, 16)]
    # host loop (GPT.generate with top_k = 1)
    host_ids = list(gpt.generate(prompt, 12, 1, 1.0))
    # oracle loop: full-window recompute per token, as the reference does
    hist = list(prompt)
    for i in range(12):
        lg = ref.forward(p, w, np.array(hist, np.int32))
        nxt = int(np.argmax(lg))
        if nxt != host_ids[i]:
            assert greedy_ok(gpt.run(hist), lg)
            break
        hist.append(nxt)
    # device loop: prefill, then all steps on the device
    lg = gpt.prefill(prompt)
    first = int(np.argmax(lg))
    dev_ids, last_logits = gpt.decode_greedy(first, 11, want_logits=True)
    assert [first] + [int(t) for t in dev_ids] == host_ids[:12]
    gpt.unloadBuffers()


def test_context_limit_and_errors(device):
    cfg = small_cfg(n_ctx=12)
    gpt, tensors = load(cfg, seed=2)
    tokens = synth.tokens(3, "prompt", 12, cfg["vocab_size"])
    gpt.prefill(tokens[:11])
    gpt.decode(int(tokens[11]))
    with pytest.raises(WgptError, match="context"):
        gpt.decode(1)
    with pytest.raises(WgptError, match="outside"):
        gpt.prefill([cfg["vocab_size"]])
    with pytest.raises(WgptError, match="exceeds"):
        gpt.prefill(np.zeros(13, np.int32))
    # sliding the window (model.js:69): recompute on the last n_ctx tokens, positions restart at 0
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    hist = list(tokens) + [5, 6]
    got = gpt.run(hist[-12:])
    assert close(got, ref.forward(p, w, np.array(hist[-12:], np.int32)))
    gpt.unloadBuffers()


def test_int8_model(device):
    cfg = small_cfg(n_layer=2, n_head=2, n_embd=64, n_ctx=24, vocab_size=50, dtype="int8")
    gpt, tensors = load(cfg, seed=13)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(3, "prompt", 12, cfg["vocab_size"])
    for T in (3, 9):      # GEMV path (<= 4 rows) and the dequantise + GEMM path
        got = gpt.prefill(tokens[:T])
        want = ref.forward(p, w, tokens[:T])
        assert close(got, want), worst(got, want)
    got = gpt.run(tokens[:10])
    want = ref.forward(p, w, tokens[:10])
    assert close(got, want), worst(got, want)
    gpt.unloadBuffers()


def test_gpt2_117m_shape_prefill_and_decode(device):
    cfg = dict(synth.CONFIGS["gpt2-117m"])
    gpt, tensors = load(cfg, seed=1, random_ln=False)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.make_prompt(cfg, 1, 24)
    got = gpt.prefill(tokens[:20])
    want = ref.forward(p, w, tokens[:20])
    assert close(got, want), worst(got, want)
    for t in range(20, 24):
        got = gpt.decode(int(tokens[t]))
    want = ref.forward(p, w, tokens[:24])
    assert close(got, want), worst(got, want)
    assert greedy_ok(got, want)
    assert gpt.decode_bytes(0) == 4 * (12 * (12 * 768 * 768 + 13 * 768) + 50257 * 768 + 2 * 768)
    gpt.unloadBuffers()


@pytest.mark.parametrize("name,steps", [("toy", 40), ("gpt2-117m", 6)])
def test_persistent_decode_matches_per_block_decode_and_oracle(device, name, steps):
    # decode mode 1 (one persistent kernel per token) against mode 0 (one kernel per block) and the oracle
    cfg = dict(synth.CONFIGS[name])
    gpt, tensors = load(cfg, seed=5, random_ln=(name == "toy"))
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(8, "prompt", 10 + steps, cfg["vocab_size"])
    out = {}
    for mode in (0, 1):
        gpt.set_decode_mode(mode)
        gpt.prefill(tokens[:10])
        out[mode] = [gpt.decode(int(tokens[10 + i])) for i in range(steps)]
    for i in range(steps):
        assert close(out[1][i], out[0][i]), (i, worst(out[1][i], out[0][i]))
    for i in (0, steps - 1):
        want = ref.forward(p, w, tokens[: 11 + i])
        assert close(out[1][i], want), (i, worst(out[1][i], want))
        assert greedy_ok(out[1][i], want)
    # the cache written by the persistent kernel serves the per-block path and vice versa
    gpt.set_decode_mode(1)
    gpt.prefill(tokens[:10])
    a = gpt.decode(int(tokens[10]))
    gpt.set_decode_mode(0)
    b = gpt.decode(int(tokens[11]))
    assert close(a, out[0][0]) and close(b, out[0][1])
    # multi-step greedy launch: ids equal the per-block greedy loop
    ids = {}
    for mode in (0, 1):
        gpt.set_decode_mode(mode)
        lg = gpt.prefill(tokens[:10])
        ids[mode] = [int(t) for t in gpt.decode_greedy(int(np.argmax(lg)), min(steps, 24))]
    assert ids[0] == ids[1]
    gpt.unloadBuffers()


def test_poll_delay_search_changes_timing_only(device):
    # wgpt_model_tune_poll_delays: the row it keeps is no slower than the one it started from (as it measured them),
    # logits and greedy ids of a context decoded afterwards are those of a model that never searched, and it refuses
    # to run while a context is in use
    cfg = dict(synth.CONFIGS["toy"])
    gpt, tensors = load(cfg, seed=5)
    tokens = synth.tokens(8, "prompt", 12, cfg["vocab_size"])
    lg = gpt.prefill(tokens)
    want_ids = [int(t) for t in gpt.decode_greedy(int(np.argmax(lg)), 30)]
    gpt.prefill(tokens[:11])
    want_logits = gpt.decode(int(tokens[11]))
    with pytest.raises(WgptError, match="context is in use"):
        gpt.tune_poll_delays(1)
    _lib.call("wgpt_model_reset_cache", gpt._handle)
    start = gpt.poll_delays()
    row, before, after = gpt.tune_poll_delays(1)
    print("poll delays", start, "->", row, "ms/token", before, "->", after)
    assert len(row) == 7 and all(0 <= v <= 1024 for v in row) and row == gpt.poll_delays()
    assert 0 < after <= before
    lg = gpt.prefill(tokens)
    assert [int(t) for t in gpt.decode_greedy(int(np.argmax(lg)), 30)] == want_ids
    gpt.prefill(tokens[:11])
    assert np.array_equal(gpt.decode(int(tokens[11])), want_logits)
    gpt.unloadBuffers()
    # the same search as the last step of wgpt_model_finalize
    gpt2, _ = load(cfg, seed=5, flags=_lib.FLAG_TUNE_DELAYS)
    lg = gpt2.prefill(tokens)
    assert [int(t) for t in gpt2.decode_greedy(int(np.argmax(lg)), 30)] == want_ids
    gpt2.unloadBuffers()


@pytest.mark.parametrize("start", [2**31 - 1 - 60, 2**31 - 1 - 1000, 2**31 - 1 - 1500])
def test_epoch_counter_restarts_below_its_limit(device, monkeypatch, start):
    # the exchange words carry a 32-bit epoch that only grows; a model that has decoded for hours reaches the
    # limit, clears its exchange buffers and starts over. Started just below the limit (at once, within the first
    # greedy call, within the third), the tokens and logits are those of a counter that starts at 0.
    cfg = dict(synth.CONFIGS["toy"])
    cfg["n_layer"] = 3
    tokens = synth.tokens(8, "prompt", 12, cfg["vocab_size"])
    runs = {}
    for s0 in (0, start):
        if s0:
            monkeypatch.setenv("WEBGPT_AMD_EPOCH_START", str(s0))
        else:
            monkeypatch.delenv("WEBGPT_AMD_EPOCH_START", raising=False)
        gpt, _ = load(cfg, seed=5)
        lg = gpt.prefill(tokens)
        ids = [int(t) for t in gpt.decode_greedy(int(np.argmax(lg)), 40)]
        ids += [int(t) for t in gpt.decode_greedy(ids[-1], 40)]
        ids += [int(t) for t in gpt.decode_greedy(ids[-1], 40)]
        last = gpt.decode(ids[-1])
        runs[s0] = (ids, last.copy())
        gpt.unloadBuffers()
    assert runs[start][0] == runs[0][0]
    assert np.array_equal(runs[start][1], runs[0][1])


def test_two_models_decode_interleaved(device):
    # two models alive at once (their own caches, exchange buffers and epochs), their decode calls interleaved:
    # each gives what it gives alone
    cfg = dict(synth.CONFIGS["toy"])
    cfg["n_layer"] = 2
    tokens = synth.tokens(8, "prompt", 10, cfg["vocab_size"])
    alone = {}
    for seed in (5, 6):
        gpt, _ = load(cfg, seed=seed)
        lg = gpt.prefill(tokens)
        first = int(np.argmax(lg))
        ids = [int(t) for t in gpt.decode_greedy(first, 9)]
        alone[seed] = (first, ids, gpt.decode(ids[-1]).copy())
        gpt.unloadBuffers()
    a, _ = load(cfg, seed=5)
    b, _ = load(cfg, seed=6)
    la, lb = a.prefill(tokens), b.prefill(tokens)
    fa, fb = int(np.argmax(la)), int(np.argmax(lb))
    ia, ib = [], []
    ta, tb = fa, fb
    for _ in range(3):   # three calls of three steps each, alternating
        ia += [int(t) for t in a.decode_greedy(ta, 3)]
        ib += [int(t) for t in b.decode_greedy(tb, 3)]
        ta, tb = ia[-1], ib[-1]
    assert (fa, ia) == alone[5][:2] and (fb, ib) == alone[6][:2]
    assert np.array_equal(b.decode(ib[-1]), alone[6][2]) and np.array_equal(a.decode(ia[-1]), alone[5][2])
    a.unloadBuffers()
    b.unloadBuffers()


@pytest.mark.parametrize("name", ["gpt2-345m", "gpt2-774m"])
def test_larger_shapes_decode_against_oracle(device, name):
    # the persistent decode kernel is instantiated per model width; check the other widths too
    cfg = dict(synth.CONFIGS[name])
    cfg["n_layer"] = 4          # same width/heads/vocab, fewer layers: keeps the oracle run short
    gpt, tensors = load(cfg, seed=2, random_ln=True)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(6, "prompt", 14, cfg["vocab_size"])
    got = gpt.prefill(tokens[:9])
    want = ref.forward(p, w, tokens[:9])
    assert close(got, want), worst(got, want)
    out = {}
    for mode in (0, 1):
        gpt.set_decode_mode(mode)
        gpt.prefill(tokens[:9])
        out[mode] = [gpt.decode(int(tokens[9 + i])) for i in range(5)]
    want = ref.forward(p, w, tokens)
    for mode in (0, 1):
        assert close(out[mode][-1], want), (mode, worst(out[mode][-1], want))
    assert greedy_ok(out[1][-1], want)
    gpt.unloadBuffers()


@pytest.mark.parametrize("name,n_layer", [("gpt2-117m", 2), ("gpt2-345m", 2)])
def test_multi_step_launch_logits_equal_single_step_launches(device, name, n_layer):
    # A launch of several steps keeps part of the vocabulary table on the chip (LDS, registers) and reads the rest
    # from memory; a single-step launch reads all of it from memory. Same sums, same order: the logits of the last
    # step are the same bits, and so is every chosen token (full 50257-row table, so every workgroup has a full run).
    cfg = dict(synth.CONFIGS[name])
    cfg["n_layer"] = n_layer
    gpt, _ = load(cfg, seed=21, random_ln=True)
    gpt.set_decode_mode(1)
    tokens = synth.tokens(5, "prompt", 40, cfg["vocab_size"])
    first = int(np.argmax(gpt.prefill(tokens)))
    ids, last = gpt.decode_greedy(first, 6, want_logits=True)
    gpt.prefill(tokens)
    tok, single = first, []
    for _ in range(6):
        lg = gpt.decode(tok)
        tok = int(np.argmax(lg))
        single.append(tok)
    assert [int(t) for t in ids] == single
    assert np.array_equal(last, lg)
    gpt.unloadBuffers()


@pytest.mark.parametrize("name,n_layer", [("toy", 3), ("gpt2-117m", 2)])
def test_persistent_decode_across_the_short_context_limit(device, name, n_layer):
    # the persistent kernel exists per context range (up to 512 positions, and beyond): steps on both sides of
    # the limit, and multi-step launches that cross it, against the per-block path
    cfg = dict(synth.CONFIGS[name])
    cfg["n_layer"], cfg["n_ctx"] = n_layer, 1024
    gpt, tensors = load(cfg, seed=9, random_ln=True)
    tokens = synth.tokens(12, "prompt", 540, cfg["vocab_size"])
    out, ids, sampled, last = {}, {}, {}, {}
    u = np.random.default_rng(3).random(16)
    for mode in (0, 1):
        gpt.set_decode_mode(mode)
        gpt.prefill(tokens[:505])
        out[mode] = [gpt.decode(int(tokens[505 + i])) for i in range(14)]       # contexts 506..519
        lg = gpt.prefill(tokens[:500])
        got, last[mode] = gpt.decode_greedy(int(np.argmax(lg)), 24, want_logits=True)   # one call, contexts 501..524
        ids[mode] = [int(t) for t in got]
        gpt.prefill(tokens[:504])
        sampled[mode] = [int(t) for t in gpt.decode_sample(int(tokens[504]), len(u), 4, 0.9, u)]
    for i in range(14):
        assert close(out[1][i], out[0][i]), (i, worst(out[1][i], out[0][i]))
    # both context ranges of the persistent kernel against the oracle itself: the full forward over the history
    # (model.js:104-241) at a context below the limit of 512 positions and at one above it
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    for i in (0, 13):                                                            # contexts 506 and 519
        want = ref.forward(p, w, tokens[:506 + i])
        for mode in (1, 0):
            assert close(out[mode][i], want), (name, mode, 506 + i, worst(out[mode][i], want))
        assert greedy_ok(out[1][i], want)
    assert ids[0] == ids[1]
    # (the second of the call's two launches hands its logits to the host itself)
    assert close(last[1], last[0]), worst(last[1], last[0])
    assert sampled[0] == sampled[1]
    gpt.unloadBuffers()


def test_model_create_refuses_what_the_decode_kernels_cannot_stage(device):
    # the reference's load checks (model.js:294-297) and the library's own limits, before any tensor is uploaded
    def create(**kw):
        p = dict(n_layer=1, n_head=2, n_embd=128, n_ctx=16, vocab_size=40, weight_dtype=0, max_prefill=0, flags=0)
        p.update(kw)
        h = C.c_uint64(0)
        _lib.call("wgpt_model_create", C.byref(_lib.Params(**p)), C.byref(h))
        _lib.call("wgpt_model_destroy", h.value)
    create()
    create(n_head=48, n_embd=3072)
    with pytest.raises(WgptError, match="n_embd above 3072"):
        create(n_head=49, n_embd=3136)
    with pytest.raises(WgptError, match="n_embd must be divisible by n_head"):
        create(n_head=3, n_embd=128)
    with pytest.raises(WgptError, match="head size above 256"):
        create(n_head=1, n_embd=512)


def test_external_buffer_receives_the_last_residual_rows(device):
    # model.js:211-222: with GPT.externalBuffer set (visuals.js:48-50) run() copies the residual stream after the
    # last layer, [seq_length, n_embd], into it
    from webgpt_amd.blocks import Buffer
    cfg = dict(synth.CONFIGS["toy"])
    cfg["n_layer"] = 2
    gpt, tensors = load(cfg, seed=31)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(8, "prompt", 21, cfg["vocab_size"])
    plain = [gpt.run(tokens[:20]), gpt.run(tokens)]          # prefill, then a cached step
    gpt.externalBuffer = Buffer([cfg["n_ctx"], cfg["n_embd"]])
    for T in (20, 21):
        want_logits, want_taps, _ = ref.forward(p, w, tokens[:T], want_taps=True, want_kv=True)
        logits = gpt.run(tokens[:T])
        rows = gpt.externalBuffer.download(count=T * cfg["n_embd"]).reshape(T, cfg["n_embd"])
        want = want_taps[ref.tap_names(cfg["n_layer"]).index(f"block{cfg['n_layer'] - 1}_r2")]
        assert close(rows, want), worst(rows, want)
        assert close(logits, want_logits) and close(logits, plain[T - 20])
    gpt.externalBuffer.destroy()
    gpt.externalBuffer = None
    gpt.unloadBuffers()


def test_int8_persistent_decode_against_oracle(device):
    # width of the 1.5B int8 configuration, two layers: persistent int8 decode vs per-block int8 decode vs oracle
    cfg = dict(synth.CONFIGS["gpt2-1.5b-int8"])
    cfg["n_layer"] = 2
    gpt, tensors = load(cfg, seed=4, random_ln=True)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(6, "prompt", 13, cfg["vocab_size"])
    out = {}
    for mode in (0, 1):
        gpt.set_decode_mode(mode)
        gpt.prefill(tokens[:8])
        out[mode] = [gpt.decode(int(tokens[8 + i])) for i in range(5)]
    want = ref.forward(p, w, tokens)
    for mode in (0, 1):
        assert close(out[mode][-1], want), (mode, worst(out[mode][-1], want))
    assert greedy_ok(out[1][-1], want)
    gpt.unloadBuffers()


def test_expired_wait_disables_the_persistent_path_and_falls_back(device, monkeypatch):
    """A bounded wait of the persistent kernel that expires (forced from the host: no delay before the
    first look and no further round after it, so every workgroup gives up at once and the launch
    drains normally) is reported as an error, and decoding continues on the per-block kernels with
    correct results."""
    cfg = small_cfg(n_layer=2, n_head=6, n_embd=384, n_ctx=32, vocab_size=90)
    monkeypatch.setenv("WEBGPT_AMD_SPIN_LIMIT", "0")             # give up at the first look that finds a word missing
    monkeypatch.setenv("WEBGPT_AMD_POLL_DELAYS", "0,0,0,0,0,0,0")  # and look at once, before any other workgroup can have published
    gpt, tensors = load(cfg, seed=17)
    monkeypatch.delenv("WEBGPT_AMD_SPIN_LIMIT")
    monkeypatch.delenv("WEBGPT_AMD_POLL_DELAYS")
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(17, "prompt", 10, cfg["vocab_size"])
    gpt.prefill(tokens[:8])
    with pytest.raises(WgptError, match="bounded wait expired"):
        gpt.decode(int(tokens[8]))
    with pytest.raises(WgptError, match="not available"):
        gpt.set_decode_mode(1)
    got = gpt.decode(int(tokens[8]))                  # same token again, now on the per-block path
    assert close(got, ref.forward(p, w, tokens[:9])), worst(got, ref.forward(p, w, tokens[:9]))
    got = gpt.decode(int(tokens[9]))
    assert close(got, ref.forward(p, w, tokens[:10]))
    gpt.unloadBuffers()


@pytest.mark.parametrize("top_k", [3, 12])
def test_expired_wait_in_decode_sample_leaves_the_position_unchanged(device, monkeypatch, top_k):
    """The same host-forced expiry (every kernel exits normally) met by wgpt_decode_sample, on its in-kernel
    selection (top_k <= 8) and on its one-launch-per-token loop: the call fails, the cache position is what it
    was before the call, and a retry of the same tokens, now on the per-block kernels, gives the oracle's result."""
    cfg = small_cfg(n_layer=2, n_head=6, n_embd=384, n_ctx=32, vocab_size=90)
    monkeypatch.setenv("WEBGPT_AMD_SPIN_LIMIT", "0")
    monkeypatch.setenv("WEBGPT_AMD_POLL_DELAYS", "0,0,0,0,0,0,0")
    gpt, tensors = load(cfg, seed=19)
    monkeypatch.delenv("WEBGPT_AMD_SPIN_LIMIT")
    monkeypatch.delenv("WEBGPT_AMD_POLL_DELAYS")
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(19, "prompt", 9, cfg["vocab_size"])
    gpt.prefill(tokens[:8])
    u = np.array([0.3, 0.6, 0.9])
    with pytest.raises(WgptError, match="bounded wait expired"):
        gpt.decode_sample(int(tokens[8]), 3, top_k, 0.8, u)
    pos = C.c_int(-1)
    _lib.call("wgpt_model_position", gpt._handle, C.byref(pos))
    assert pos.value == 8
    assert gpt._history == [int(t) for t in tokens[:8]]
    # retry: same token, same draws, per-block kernels; the oracle's loop (model.js:81-85) over full forwards
    got = [int(t) for t in gpt.decode_sample(int(tokens[8]), 3, top_k, 0.8, u)]
    hist = [int(t) for t in tokens[:9]]
    for i in range(3):
        lg = ref.forward(p, w, np.array(hist, np.int32))
        nxt, _, _ = ref.sample_topk(lg, top_k, 0.8, float(u[i]))
        assert got[i] == nxt, (i, got, nxt)
        hist.append(nxt)
    _lib.call("wgpt_model_position", gpt._handle, C.byref(pos))
    assert pos.value == 11
    gpt.unloadBuffers()


@pytest.mark.parametrize("name,dtype", [("toy", "f32"), ("toy", "int8")])
def test_per_block_decode_graph_replays_equal_eager_launches(device, monkeypatch, name, dtype):
    """With WEBGPT_AMD_TOKEN_GRAPH=1 decode mode 0 records the launches of a token as a HIP graph (kernel nodes only; the
    position is read from device memory) and replays it for every later token. Every replay, with eager prefills,
    host loops and synchronisations between them, must give what the same launches give when issued one by one (the
    default), bit for bit, and both must match the oracle."""
    cfg = dict(synth.CONFIGS[name])
    cfg["n_layer"], cfg["dtype"] = 3, dtype
    tokens = synth.tokens(31, "prompt", 40, cfg["vocab_size"])
    out = {}
    for graph in (True, False):
        if graph:
            monkeypatch.setenv("WEBGPT_AMD_TOKEN_GRAPH", "1")
        gpt, tensors = load(cfg, seed=29)
        gpt.set_decode_mode(0)
        res = []
        gpt.prefill(tokens[:9])
        res += [gpt.decode(int(tokens[9 + i])) for i in range(6)]            # six replays, a read-back after each
        ids = gpt.decode_greedy(int(tokens[15]), 5)                          # five replays in one call
        res.append(np.asarray(ids, np.float32))
        gpt.prefill(tokens[:20])                                             # eager work in between
        res += [gpt.decode(int(tokens[20 + i])) for i in range(4)]
        res.append(np.asarray(gpt.decode_sample(int(tokens[24]), 4, 3, 0.9, np.array([0.1, 0.5, 0.7, 0.95])), np.float32))
        out[graph] = res
        if graph:
            w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
            want = ref.forward(p, w, tokens[:24])
            assert close(res[10], want), worst(res[10], want)
        gpt.unloadBuffers()
        monkeypatch.delenv("WEBGPT_AMD_TOKEN_GRAPH", raising=False)
    assert len(out[True]) == len(out[False])
    for i, (a, b) in enumerate(zip(out[True], out[False])):
        assert np.array_equal(a, b), i


@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("n_head,n_embd,n_ctx,start", [(2, 128, 600, 250), (3, 96, 1100, 1020)])
def test_per_block_decode_across_cache_slices(device, monkeypatch, graph, n_head, n_embd, n_ctx, start):
    """Decode mode 0 attends with a workgroup per (head, slice of the cache: 64 positions at head size 64, 128 at 32)
    and merges the slices in the attention projection; the slices the host expects to hold positions request their
    rows early, the others look at the position first. Steps on both sides of slice boundaries (and of the end of
    a cache that is not a whole number of slices), issued one by one and replayed as a graph (which expects only
    the first slice), against the oracle's full forward over the history (model.js:104-241)."""
    cfg = small_cfg(n_layer=2, n_head=n_head, n_embd=n_embd, n_ctx=n_ctx, vocab_size=97)
    if graph:
        monkeypatch.setenv("WEBGPT_AMD_TOKEN_GRAPH", "1")
    gpt, tensors = load(cfg, seed=37)
    gpt.set_decode_mode(0)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(41, "prompt", start + 12, cfg["vocab_size"])
    gpt.prefill(tokens[:start])
    for i in range(12):
        got = gpt.decode(int(tokens[start + i]))
        if i in (0, 3, 4, 5, 6, 11):  # hs 64: position 256 starts a slice; hs 32: position 1024 does
            want = ref.forward(p, w, tokens[:start + i + 1])
            assert close(got, want), (i, worst(got, want))
    ids = gpt.decode_greedy(int(np.argmax(got)), 3)
    hist = [int(t) for t in tokens[:start + 12]] + [int(np.argmax(got))]
    for t in ids:
        lg = ref.forward(p, w, np.array(hist, np.int32))
        assert int(np.argmax(lg)) == int(t) or greedy_gap_ok(lg, int(t)), (int(np.argmax(lg)), int(t))
        hist.append(int(t))
    gpt.unloadBuffers()


def greedy_gap_ok(logits, chosen):
    best = int(np.argmax(logits))
    return abs(float(logits[best] - logits[chosen])) <= 1e-5 + 1e-4 * abs(float(logits[best]))
