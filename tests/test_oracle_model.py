"""Pins the oracle's whole-model forward (GPT.run restatement) against a textbook
GPT-2 forward built from torch library routines in float64 (tests/gpt2_torch.py),
tap by tap with the reference's validation names."""
import numpy as np
import pytest

from oracle import ref
from webgpt_amd import synth

import gpt2_torch
from helpers import close, make_model, oracle_weights, small_cfg, worst


@pytest.mark.parametrize("cfg,T", [
    (small_cfg(), 1), (small_cfg(), 11), (small_cfg(n_layer=3, n_head=4, n_embd=64, n_ctx=40, vocab_size=97), 40),
    (dict(synth.CONFIGS["toy"]), 24),
])
def test_forward_taps_and_logits_vs_torch(cfg, T):
    tensors = make_model(cfg, seed=11)
    tokens = synth.tokens(5, "prompt", T, cfg["vocab_size"])
    logits, taps, kv = ref.forward(synth.model_params(cfg), oracle_weights(tensors, cfg), tokens,
                                   want_taps=True, want_kv=True)
    want_logits, want = gpt2_torch.forward(cfg, tensors, tokens)
    for i, name in enumerate(ref.tap_names(cfg["n_layer"])):
        assert close(taps[i], want[name].numpy()), (name, worst(taps[i], want[name].numpy()))
    for i in range(cfg["n_layer"]):
        assert close(kv[i, 0], want[f"kv{i}_k"].numpy()) and close(kv[i, 1], want[f"kv{i}_v"].numpy())
    assert close(logits, want_logits.numpy()), worst(logits, want_logits.numpy())
    assert int(np.argmax(logits)) == int(np.argmax(want_logits.numpy()))


def test_forward_is_causal_last_row_of_prefix():
    # the logits for window [0..t] do not depend on later tokens: the property the
    # KV-cache decode path relies on
    cfg = small_cfg()
    tensors = make_model(cfg, seed=3)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(9, "prompt", 12, cfg["vocab_size"])
    _, taps_full = ref.forward(p, w, tokens, want_taps=True)
    for t in (1, 5, 12):
        _, taps_t = ref.forward(p, w, tokens[:t], want_taps=True)
        assert np.array_equal(taps_t[:, :t], taps_full[:, :t])


def test_forward_rejects_bad_arguments():
    cfg = small_cfg()
    tensors = make_model(cfg, seed=3)
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    with pytest.raises(ValueError):
        ref.forward(p, w, np.array([cfg["vocab_size"]], np.int32))
    with pytest.raises(ValueError):
        ref.forward(p, w, np.zeros(cfg["n_ctx"] + 1, np.int32))


def test_int8_model_forward_equals_fp32_forward_on_dequantised_weights():
    cfg = small_cfg(dtype="int8")
    tensors = make_model(cfg, seed=21)
    tokens = synth.tokens(2, "prompt", 9, cfg["vocab_size"])
    got = ref.forward(synth.model_params(cfg), oracle_weights(tensors, cfg), tokens)
    deq = {}
    for name, a in tensors.items():
        if name.endswith(".weight.q"):
            stem = name[:-2]
            deq[stem] = ref.dequant_i8(a, tensors[stem + ".scale"], tensors[stem + ".scale"].shape[0])
        elif not name.endswith(".weight.scale"):
            deq[name] = a
    fcfg = dict(cfg, dtype="f32")
    want = ref.forward(synth.model_params(fcfg), oracle_weights(deq, fcfg), tokens)
    assert np.array_equal(got, want)
