"""Validation-JSON harness (other/validation/validation.js:113-134,183-222)."""
import json

import numpy as np
import pytest

from webgpt_amd import _lib, synth, validation

from helpers import make_model, oracle_weights, small_cfg


def oracle_steps(cfg, tensors, prompt, steps):
    """What a reference implementation would export: the oracle's taps per greedy step."""
    from oracle import ref
    p, w = synth.model_params(cfg), oracle_weights(tensors, cfg)
    hist = [int(t) for t in prompt]
    out = []
    for _ in range(steps):
        logits, taps = ref.forward(p, w, np.array(hist, np.int32), want_taps=True)
        step = {n: {"shape": [1] + list(taps[i].shape), "data": [taps[i].tolist()]} for i, n in enumerate(ref.tap_names(cfg["n_layer"]))}
        step["logits"] = {"shape": [1, 1, logits.size], "data": [[logits.tolist()]]}
        out.append(step)
        hist.append(int(np.argmax(logits)))
    return out


def test_schema_round_trip(tmp_path):
    cfg = small_cfg()
    steps = oracle_steps(cfg, make_model(cfg, 2), [1, 2, 3], 2)
    assert validation.tap_names(cfg["n_layer"]) == [k for k in steps[0] if k != "logits"]
    path = tmp_path / "v.json"
    path.write_text(json.dumps(steps))
    loaded = validation.load(str(path))
    assert len(loaded) == 2
    assert loaded[0]["tok_pos_emb"].shape == (1, 3, cfg["n_embd"]) and loaded[1]["block1_r2"].shape == (1, 4, cfg["n_embd"])
    assert loaded[0]["logits"].shape == (1, 1, cfg["vocab_size"]) and loaded[0]["logits"].dtype == np.float32
    bad = [{"ln_f": {"shape": [1, 2, 2], "data": [[1.0, 2.0, 3.0]]}}]
    with pytest.raises(ValueError, match="ln_f"):
        validation.load(bad)


@pytest.mark.gpu
def test_validate_and_dump_on_gpu(device, tmp_path):
    from webgpt_amd.model import GPT
    cfg = small_cfg(n_layer=2, n_head=2, n_embd=128, n_ctx=16, vocab_size=80)
    tensors = make_model(cfg, 4)
    prompt = [int(t) for t in synth.tokens(4, "prompt", 5, cfg["vocab_size"])]
    steps = oracle_steps(cfg, tensors, prompt, 3)
    gpt = GPT(None, "char", tensors=tensors, params=synth.model_params(cfg), flags=_lib.FLAG_TAPS)
    gpt.initialize()
    try:
        assert validation.validate(gpt, steps, prompt) == []
        # a reference that disagrees in one activation is reported by step and name
        steps[1]["block1_mlp"]["data"][0][2][7] += 0.01
        fails = validation.validate(gpt, steps, prompt)
        assert [(s, k) for s, k, _ in fails] == [(1, "block1_mlp")]
        # dump writes the same schema and validates against itself
        mine = validation.dump(gpt, prompt, 2, str(tmp_path / "mine.json"))
        assert sorted(mine[0]) == sorted(steps[0]) and mine[1]["ln_f"]["shape"] == [1, 6, cfg["n_embd"]]
        assert validation.validate(gpt, str(tmp_path / "mine.json"), prompt, tolerance=0.0) == []
    finally:
        gpt.unloadBuffers()
