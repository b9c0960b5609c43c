"""The C-ABI library loads, exports every symbol include/webgpt_amd.h declares, and
refuses to compute without a device (no CPU fallback). No GPU needed."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from webgpt_amd import WgptError, _lib, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "webgpt_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wgpt_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    lib = _lib.cdll()
    names = declared_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(names) == _lib.EXPORTS


def test_product_never_touches_the_oracle():
    # nothing under webgpt_amd/ may import, link or load anything from oracle/
    bad = []
    for dirpath, _, files in os.walk(os.path.join(ROOT, "webgpt_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp", ".cc", ".js", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                if re.search(r"oracle", text):
                    bad.append(os.path.join(dirpath, f))
    assert not bad, bad


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_compute_fails_loudly_without_a_device():
    with pytest.raises(WgptError, match="no CPU fallback"):
        _lib.init(0)
    h = C.c_uint64(0)
    with pytest.raises(WgptError, match="wgpt_init"):
        _lib.call("wgpt_alloc", 16, C.byref(h))
    with pytest.raises(WgptError, match="wgpt_init"):
        _lib.call("wgpt_matmul_bias", 1, 8, 4, 1, 2, 3, 4)


def test_synth_c_equals_numpy():
    for name, n in (("transformer.wte.weight", 3000), ("transformer.h.3.mlp.c_fc.bias", 17)):
        a = synth.normal(7, name, (n,))
        assert np.array_equal(a, synth.normal_np(7, synth.tensor_id(name), n))
    a = synth.normal(1, "big", (200000,))
    assert abs(float(a.std()) - 0.02) < 2e-4 and abs(float(a.mean())) < 2e-4
    assert np.array_equal(synth.tokens(3, "prompt", 500, 50257), synth.tokens_np(3, synth.tensor_id("prompt"), 500, 50257))
    q = synth.int8_packed(3, "x.q", 8, 16)
    vals = synth.int8_np(3, synth.tensor_id("x.q"), 128)
    assert np.array_equal(q, synth.pack_int8(vals, 8, 16)) and vals.min() >= -127 and vals.max() <= 127
    s = synth.uniform(3, "s", 999, 1e-3, 1e-2)
    assert np.array_equal(s, synth.uniform_np(3, synth.tensor_id("s"), 999, 1e-3, 1e-2))
    assert s.min() >= np.float32(1e-3) and s.max() < np.float32(1e-2)
    assert _lib.cdll().wgpt_synth_tensor_id(b"prompt") == synth.tensor_id("prompt")


def test_config_table_matches_baseline_shapes():
    c = synth.CONFIGS["gpt2-117m"]
    assert (c["n_layer"], c["n_head"], c["n_embd"], c["n_ctx"], c["vocab_size"], c["prompt"], c["decode"]) == \
        (12, 12, 768, 1024, 50257, 128, 256)
    n = sum(int(np.prod(s)) for _, s, _ in synth.tensor_shapes(c))
    assert n * 4 == 4 * (12 * (12 * 768 * 768 + 13 * 768) + 50257 * 768 + 2 * 768) + 4 * 1024 * 768
