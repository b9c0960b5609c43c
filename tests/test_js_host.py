"""The JavaScript host (webgpt_amd/js: GPT, instruction blocks, globals, N-API addon)."""
import json
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from webgpt_amd import synth

from helpers import close, oracle_weights, worst

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NODE = shutil.which("node")
pytestmark = pytest.mark.skipif(NODE is None, reason="node is not installed")


def run_node(script, *args, timeout=120):
    r = subprocess.run([NODE, os.path.join(ROOT, "tests", "js", script), *args], capture_output=True, text=True, timeout=timeout, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    return json.loads(r.stdout.strip().splitlines()[-1])


def test_host_functions_and_generator_without_gpu():
    out = run_node("host_checks.js")
    # the addon binds every symbol the header declares
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "webgpt_amd.h")).read(), flags=re.S)
    assert sorted(out["exports"]) == sorted(set(re.findall(r"\b(wgpt_[a-z0-9_]+)\s*\(", text)))
    # the reference's global names exist (globals.js:1-27, instructions.js, model.js)
    for n in ("GPT", "FastMatMulBlock", "AttentionBlock", "ResidualBlock", "EmbedBlock", "DeEmbedBlock", "GeluBlock", "LayerNormBlock",
              "SoftmaxBlock", "initializeOperations", "destroyOperationBuffers", "clearOperationCache", "destroyOperations",
              "bufferUsageDict", "wgSize", "sampleFromDistribution", "cpuSoftmax", "selectTopK", "transpose", "zeros", "formatAsMatrix"):
        assert n in out["names"], n
    # generator: JavaScript == C == numpy, bit for bit
    name = "transformer.h.3.mlp.c_fc.bias"
    want = synth.normal(7, name, (64,))
    assert np.array_equal(np.array(out["normal"], np.float32), want)
    assert np.array_equal(np.array(out["nativeNormal"], np.float32), want)
    assert out["tokens"] == [int(t) for t in synth.tokens(3, "prompt", 64, 50257)]
    assert np.array_equal(np.array(out["int8"], np.int64).astype(np.int32), synth.int8_packed(3, "x.q", 8, 16).ravel())
    assert np.array_equal(np.array(out["uniform"], np.float32), synth.uniform(3, "s", 33, 1e-3, 1e-2))
    assert out["tensorId"] == synth.tensor_id("transformer.wte.weight")
    # selectTopK: stable descending sort, ties keep the lower index (globals.js:66-74)
    assert out["topk"]["topKIndices"] == [1, 3, 4] and out["topk"]["topKProbs"] == [2.0, 2.0, 1.5]
    assert out["top1"]["topKIndices"] == [1]
    e = np.exp((np.array([1.0, 2.0, 4.0]) - 4.0) / 0.5)
    assert np.allclose(out["softmax"], e / e.sum(), rtol=1e-15)
    assert out["sample"] == [0, 0, 1, 1, 2, 2]          # rand < cumulative
    assert out["transpose"] == [1, 4, 2, 5, 3, 6]
    assert out["wgSize"] == [3, 2]
    # the reference's precondition messages
    assert out["errors"]["matmul"] == "Cols must be divisible by 16."
    assert out["errors"]["residual"] == out["errors"]["layernorm"] == out["errors"]["gelu"] == "Cols must be divisible by 4."
    assert out["errors"]["bufferSize"] == "Buffer size exceeds GPU limit."
    if not os.path.exists("/dev/kfd"):
        assert "no CPU fallback" in out["errors"]["device"]


@pytest.mark.gpu
def test_js_gpt_on_gpu_matches_oracle():
    from oracle import ref
    out = run_node("gpu_run.js", "toy", timeout=300)
    cfg = dict(synth.CONFIGS["toy"])
    tensors = dict(synth.make_tensors(cfg, 1))
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    tokens = synth.tokens(1, "prompt", 24, cfg["vocab_size"])
    assert out["tokens"] == [int(t) for t in tokens]
    want16, want24 = ref.forward(p, w, tokens[:16]), ref.forward(p, w, tokens)
    for key, want in (("logits16", want16), ("logits24", want24), ("blocks24", want24)):
        got = np.array(out[key], np.float32)
        assert close(got, want), (key, worst(got, want))
    got = np.array(out["chunked24"], np.float32)
    assert np.array_equal(got, np.array(out["blocks24"], np.float32))        # chunked table: same logits bit for bit
    x = np.array([[0, 1, 2], [3, 1, 1]], np.float32)
    assert np.allclose(np.array(out["softmaxT"]).reshape(3, 2), ref.softmax(x).T, rtol=1e-6, atol=1e-7)
    want20, taps20, _ = ref.forward(p, w, tokens[:20], want_taps=True, want_kv=True)
    rows = np.array(out["extRows"], np.float32).reshape(20, cfg["n_embd"])
    want_rows = taps20[ref.tap_names(cfg["n_layer"]).index(f"block{cfg['n_layer'] - 1}_r2")]
    assert close(rows, want_rows), worst(rows, want_rows)
    assert close(np.array(out["extLogits"], np.float32), want20)
    assert "outside" in out["badToken"]
    assert out["generated"] == out["greedy"]
    hist = [int(t) for t in tokens[:8]]
    for i in range(3):
        nxt = int(np.argmax(ref.forward(p, w, np.array(hist, np.int32))))
        assert nxt == out["generated"][i]
        hist.append(nxt)
    # generate() in bursts: the tokens of a call per token
    assert len(out["bursts"]["1"]) == 19
    assert out["bursts"]["8"] == out["bursts"]["1"] and out["bursts"]["5"] == out["bursts"]["1"]
    # token selection on the device, through the addon (globals.js:47-74)
    want_id, want_ids, want_p = ref.sample_topk(np.array([0.5, 2.0, -1.0, 2.0, 1.5], np.float32), 3, 0.5, 0.6)
    assert out["select"]["id"] == want_id and out["select"]["topKIndices"] == [int(i) for i in want_ids]
    assert np.allclose(out["select"]["probs"], want_p, rtol=1e-12)
    hist = [int(t) for t in tokens[:8]] + [out["greedy"][0]]
    for i, u in enumerate(out["draws"]):
        lg = ref.forward(p, w, np.array(hist, np.int32))
        want, ids, pr = ref.sample_topk(lg, 4, 0.9, u)
        assert out["sampled"][i] == want or np.min(np.abs(np.cumsum(pr) - u)) < 1e-3
        hist.append(out["sampled"][i])

