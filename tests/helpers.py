"""Shared helpers of the tests: synthetic models with non-trivial LayerNorm
parameters, the tolerance of the parity bar, packing helpers."""
import numpy as np

from webgpt_amd import synth

# Parity bar for fp32 results: |got - want| <= ATOL + RTOL * |want|.
RTOL = 1e-4
ATOL = 1e-5


def close(got, want, rtol=RTOL, atol=ATOL):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return bool(np.all(np.abs(got - want) <= atol + rtol * np.abs(want)))


def worst(got, want, rtol=RTOL, atol=ATOL):
    """Largest violation ratio |err| / (atol + rtol*|want|) (<= 1 passes)."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.max(np.abs(got - want) / (atol + rtol * np.abs(want))))


def small_cfg(n_layer=2, n_head=2, n_embd=32, n_ctx=24, vocab_size=40, dtype="f32"):
    return dict(n_layer=n_layer, n_head=n_head, n_embd=n_embd, n_ctx=n_ctx, vocab_size=vocab_size,
                prompt=8, decode=8, dtype=dtype)


def make_model(cfg, seed, random_ln=True):
    """{name: array} for a configuration. With random_ln the LayerNorm gains and
    biases are drawn too (gamma ~ 1 + N(0, 0.1), beta ~ N(0, 0.1)) so a swapped or
    dropped gamma/beta shows up; the benchmark configs themselves use gamma=1, beta=0."""
    tensors = dict(synth.make_tensors(cfg, seed))
    if random_ln:
        for name in list(tensors):
            if ".ln_" in name or "ln_f" in name:
                n = tensors[name].shape[0]
                noise = synth.normal(seed, name, (n,), 0.1)
                tensors[name] = (noise + 1.0).astype(np.float32) if name.endswith("weight") else noise
    return tensors


def pack_words(q):
    K, N = q.shape
    return synth.pack_int8(q, K, N)


def oracle_weights(tensors, cfg):
    """Regroups a {name: array} weight directory into the nested dict the CPU
    oracle's forward() takes."""
    L = cfg["n_layer"]
    w = dict(wte=tensors["transformer.wte.weight"], wpe=tensors["transformer.wpe.weight"],
             lnf_g=tensors["transformer.ln_f.weight"], lnf_b=tensors["transformer.ln_f.bias"], layers=[])
    for i in range(L):
        p = f"transformer.h.{i}."
        lw = dict(ln1_g=tensors[p + "ln_1.weight"], ln1_b=tensors[p + "ln_1.bias"],
                  ln2_g=tensors[p + "ln_2.weight"], ln2_b=tensors[p + "ln_2.bias"],
                  attn_b=tensors[p + "attn.c_attn.bias"], proj_b=tensors[p + "attn.c_proj.bias"],
                  fc_b=tensors[p + "mlp.c_fc.bias"], fc2_b=tensors[p + "mlp.c_proj.bias"])
        for key, stem in (("attn", "attn.c_attn"), ("proj", "attn.c_proj"), ("fc", "mlp.c_fc"), ("fc2", "mlp.c_proj")):
            if p + stem + ".weight" in tensors:
                lw[key + "_w"] = tensors[p + stem + ".weight"]
            else:
                lw[key + "_q"] = tensors[p + stem + ".weight.q"]
                lw[key + "_s"] = tensors[p + stem + ".weight.scale"]
        w["layers"].append(lw)
    return w
