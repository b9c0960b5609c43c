"""The weight-directory loader (model.js:270-488; format of other/conversion_scripts/*.py:
one little-endian f32 `<state_dict key>_gpt.bin` per tensor plus params_gpt.json), in
both hosts, including the two variations earlier versions of the reference read
(condensed/condensed.js:1755-1783): absent biases and [out, in] linear weights."""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

from webgpt_amd import model as wmodel
from webgpt_amd import synth

from helpers import close, make_model, oracle_weights, small_cfg, worst

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NODE = shutil.which("node")
LINEAR = ("attn.c_attn.weight", "attn.c_proj.weight", "mlp.c_fc.weight", "mlp.c_proj.weight")


def write_directory(folder, cfg, tensors, out_in=False, bias=True):
    """Writes what convert_*_pytorch.py would: returns the tensors as the forward path sees them."""
    params = synth.model_params(cfg)
    if out_in:
        params["linear_layout"] = "out_in"
    if not bias:
        params["bias"] = False
    with open(os.path.join(folder, "params_gpt.json"), "w") as f:
        json.dump(params, f)
    seen = {}
    for name, a in tensors.items():
        if name.endswith(".bias") and not bias:
            seen[name] = np.zeros_like(a)
            continue
        stored = a.T if (out_in and name.endswith(LINEAR)) else a
        np.ascontiguousarray(stored, dtype="<f4").tofile(os.path.join(folder, name + "_gpt.bin"))
        seen[name] = a
    return params, seen


@pytest.mark.parametrize("out_in,bias", [(False, True), (True, True), (True, False)])
def test_read_tensor_layouts(tmp_path, out_in, bias):
    cfg = small_cfg()
    tensors = make_model(cfg, 3)
    params, seen = write_directory(str(tmp_path), cfg, tensors, out_in, bias)
    names = list(wmodel.GPT._directory_names(params))
    assert sorted(names) == sorted(tensors)
    for n in names:
        got = wmodel.read_tensor(str(tmp_path), n, params)
        assert got.shape == tensors[n].shape == wmodel.tensor_shape(n, params), n
        assert np.array_equal(got, seen[n]), n


def test_read_tensor_rejects_wrong_size(tmp_path):
    cfg = small_cfg()
    params, _ = write_directory(str(tmp_path), cfg, make_model(cfg, 3))
    np.zeros(5, "<f4").tofile(os.path.join(str(tmp_path), "transformer.ln_f.weight_gpt.bin"))
    with pytest.raises(ValueError, match="holds 5 values, expected 32"):
        wmodel.read_tensor(str(tmp_path), "transformer.ln_f.weight", params)


@pytest.mark.skipif(NODE is None, reason="node is not installed")
@pytest.mark.parametrize("out_in,bias", [(False, True), (True, False)])
def test_js_read_tensor_layouts(tmp_path, out_in, bias):
    cfg = small_cfg()
    tensors = make_model(cfg, 5)
    params, seen = write_directory(str(tmp_path), cfg, tensors, out_in, bias)
    r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", "read_directory.js"), str(tmp_path)],
                       capture_output=True, text=True, timeout=120, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert sorted(out) == sorted(tensors)
    for n, vals in out.items():
        assert np.array_equal(np.array(vals, np.float32), seen[n].ravel()), n


@pytest.mark.gpu
@pytest.mark.parametrize("out_in,bias", [(False, True), (True, False)])
def test_gpt_from_directory_matches_oracle(device, tmp_path, out_in, bias):
    from oracle import ref
    cfg = small_cfg(n_layer=2, n_head=2, n_embd=128, n_ctx=32, vocab_size=96)
    tensors = make_model(cfg, 9)
    params, seen = write_directory(str(tmp_path), cfg, tensors, out_in, bias)
    gpt = wmodel.GPT(str(tmp_path), "char")
    gpt.initialize()
    try:
        tokens = synth.tokens(9, "prompt", 12, cfg["vocab_size"])
        got = gpt.run(tokens)
        want = ref.forward(synth.model_params(cfg), oracle_weights(seen, cfg), tokens)
        assert close(got, want), worst(got, want)
        got = gpt.run(np.append(tokens, 7))   # one more token: served from the KV cache
        want = ref.forward(synth.model_params(cfg), oracle_weights(seen, cfg), np.append(tokens, 7).astype(np.int32))
        assert close(got, want), worst(got, want)
    finally:
        gpt.unloadBuffers()
