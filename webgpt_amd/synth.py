"""Seeded synthetic models and prompts for the benchmark configurations.

Weights stand in for the reference's weight directory (one little-endian f32 file
per tensor, other/conversion_scripts/convert_pretrained_pytorch.py:18-22); tensor
names are the file stems GPT.loadModel fetches (model.js:341,371,379-383,405-420).
Values come from an integer hash of (seed, tensor name, element index), so the C
generator in the shared library, the numpy one here and the JavaScript one
(webgpt_amd/js/synth.js) agree bit for bit.
"""
import ctypes as C

import numpy as np

from . import _lib

# name -> parameters (the configurations the benchmark is defined on)
CONFIGS = {
    "toy": dict(n_layer=6, n_head=6, n_embd=384, n_ctx=256, vocab_size=65, prompt=64, decode=128, dtype="f32"),
    "gpt2-117m": dict(n_layer=12, n_head=12, n_embd=768, n_ctx=1024, vocab_size=50257, prompt=128, decode=256, dtype="f32"),
    "gpt2-345m": dict(n_layer=24, n_head=16, n_embd=1024, n_ctx=1024, vocab_size=50257, prompt=512, decode=512, dtype="f32"),
    "gpt2-774m": dict(n_layer=36, n_head=20, n_embd=1280, n_ctx=1024, vocab_size=50257, prompt=64, decode=960, dtype="f32"),
    "gpt2-1.5b": dict(n_layer=48, n_head=25, n_embd=1600, n_ctx=1024, vocab_size=50257, prompt=128, decode=256, dtype="f32"),
    "gpt2-1.5b-int8": dict(n_layer=48, n_head=25, n_embd=1600, n_ctx=1024, vocab_size=50257, prompt=128, decode=256, dtype="int8"),
}

WEIGHT_STD = 0.02
SCALE_LO, SCALE_HI = 1e-3, 1e-2

_M32 = np.uint32(0xFFFFFFFF)


def tensor_id(name):
    """FNV-1a of the tensor name (wgpt_synth_tensor_id)."""
    h = 2166136261
    for b in name.encode("utf-8"):
        h = ((h ^ b) * 16777619) & 0xFFFFFFFF
    return h


# ---- numpy restatement of webgpt_amd/csrc/wgpt_synth.h (slow; for cross-checks) ----

def _mix32(x):
    x = x.astype(np.uint32)
    x ^= x >> np.uint32(16)
    x *= np.uint32(0x7FEB352D)
    x ^= x >> np.uint32(15)
    x *= np.uint32(0x846CA68B)
    x ^= x >> np.uint32(16)
    return x


def _tensor_key(seed, tid):
    v = (seed * 0x9E3779B1 + tid * 0x85EBCA77 + 0x165667B1) & 0xFFFFFFFF
    return _mix32(np.array([v], np.uint32))[0]


def _elem_keys(tkey, index):
    index = index.astype(np.uint32)
    return _mix32(tkey ^ _mix32(index + np.uint32(0x27D4EB2F)))


def _draw(ekeys, j):
    return _mix32(ekeys + np.uint32((j * 0x9E3779B9) & 0xFFFFFFFF))


def normal_np(seed, tid, count, std=WEIGHT_STD):
    with np.errstate(over="ignore"):
        e = _elem_keys(_tensor_key(seed, tid), np.arange(count, dtype=np.uint32))
        total = np.zeros(count, np.int64)
        for j in range(12):
            total += (_draw(e, j) >> np.uint32(8)).astype(np.int64)
    total -= 6 * (1 << 24)
    return (total.astype(np.float64) * (std / 16777216.0)).astype(np.float32)


def tokens_np(seed, tid, count, vocab):
    with np.errstate(over="ignore"):
        e = _elem_keys(_tensor_key(seed, tid), np.arange(count, dtype=np.uint32))
        return (_draw(e, 0) % np.uint32(vocab)).astype(np.int32)


def int8_np(seed, tid, count):
    with np.errstate(over="ignore"):
        e = _elem_keys(_tensor_key(seed, tid), np.arange(count, dtype=np.uint32))
        return (_draw(e, 0) % np.uint32(255)).astype(np.int32) - 127


def uniform_np(seed, tid, count, lo, hi):
    with np.errstate(over="ignore"):
        e = _elem_keys(_tensor_key(seed, tid), np.arange(count, dtype=np.uint32))
        u = (_draw(e, 0) >> np.uint32(8)).astype(np.float64)
    return (lo + u * ((hi - lo) / 16777216.0)).astype(np.float32)


def pack_int8(q, K, N):
    """Packs int values in [-128,127] of a [K,N] matrix 4 per word along N
    (other/int8-gemm.js:36-43: element 0 in bits 0-7)."""
    b = (np.asarray(q, np.int64).reshape(K, N // 4, 4) & 0xFF).astype(np.uint32)
    w = b[..., 0] | (b[..., 1] << 8) | (b[..., 2] << 16) | (b[..., 3] << 24)
    return w.astype(np.uint32).view(np.int32)


# ---- fast path through the shared library ----

def normal(seed, name, shape, std=WEIGHT_STD):
    out = np.empty(shape, np.float32)
    _lib.cdll().wgpt_synth_normal(seed, tensor_id(name), out.size, std, out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def tokens(seed, name, count, vocab):
    out = np.empty(count, np.int32)
    _lib.cdll().wgpt_synth_tokens(seed, tensor_id(name), count, vocab, out.ctypes.data_as(C.POINTER(C.c_int32)))
    return out


def int8_packed(seed, name, K, N):
    out = np.empty((K, N // 4), np.int32)
    _lib.cdll().wgpt_synth_int8_packed(seed, tensor_id(name), K, N, out.ctypes.data_as(C.POINTER(C.c_int32)))
    return out


def uniform(seed, name, count, lo, hi):
    out = np.empty(count, np.float32)
    _lib.cdll().wgpt_synth_uniform(seed, tensor_id(name), count, lo, hi, out.ctypes.data_as(C.POINTER(C.c_float)))
    return out


def model_params(cfg):
    return {k: cfg[k] for k in ("n_layer", "n_head", "n_embd", "n_ctx", "vocab_size")}


def tensor_shapes(cfg):
    """(name, shape, kind) for every tensor of the weight directory. kind is one of
    normal, ones, zeros, int8 (packed words + `.scale`)."""
    d, L, V, ctx = cfg["n_embd"], cfg["n_layer"], cfg["vocab_size"], cfg["n_ctx"]
    i8 = cfg.get("dtype") == "int8"
    out = [("transformer.wte.weight", (V, d), "normal"), ("transformer.wpe.weight", (ctx, d), "normal")]
    for i in range(L):
        p = f"transformer.h.{i}."
        out += [(p + "ln_1.weight", (d,), "ones"), (p + "ln_1.bias", (d,), "zeros")]
        for stem, K, N in (("attn.c_attn", d, 3 * d), ("attn.c_proj", d, d)):
            out += [(p + stem + ".weight", (K, N), "int8" if i8 else "normal"), (p + stem + ".bias", (N,), "normal")]
        out += [(p + "ln_2.weight", (d,), "ones"), (p + "ln_2.bias", (d,), "zeros")]
        for stem, K, N in (("mlp.c_fc", d, 4 * d), ("mlp.c_proj", 4 * d, d)):
            out += [(p + stem + ".weight", (K, N), "int8" if i8 else "normal"), (p + stem + ".bias", (N,), "normal")]
    out += [("transformer.ln_f.weight", (d,), "ones"), ("transformer.ln_f.bias", (d,), "zeros")]
    return out


def make_tensors(cfg, seed):
    """Yields (name, array) for the whole weight directory of a configuration.
    int8 linear weights come as `<name>.q` (int32 words [K,N/4]) and `<name>.scale`."""
    for name, shape, kind in tensor_shapes(cfg):
        if kind == "normal":
            yield name, normal(seed, name, shape)
        elif kind == "ones":
            yield name, np.ones(shape, np.float32)
        elif kind == "zeros":
            yield name, np.zeros(shape, np.float32)
        else:
            K, N = shape
            yield name + ".q", int8_packed(seed, name + ".q", K, N)
            yield name + ".scale", uniform(seed, name + ".scale", N, SCALE_LO, SCALE_HI)


def make_prompt(cfg, seed, count=None):
    return tokens(seed, "prompt", cfg["prompt"] if count is None else count, cfg["vocab_size"])
