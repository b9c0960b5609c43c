"""GPT: the driver class of the reference's model.js over the HIP library.

`initialize()` loads a weight directory (params_gpt.json + one little-endian f32
`<tensor>_gpt.bin` per tensor, model.js:270-488) or takes tensors from memory;
`run(idx)` returns the logits of the last token of the window `idx`
(model.js:104-268); `generate()` is the sampling loop of model.js:53-102.

Two execution routes exist for `run`:
  - the whole-model entry points of the library (wgpt_prefill / wgpt_decode), which
    keep a KV cache on the device and are used whenever `idx` is the previous
    window plus one token;
  - `run_blocks(idx)`, which builds the reference's pass list block by block
    (model.js:118-240) and replays it, recomputing the whole window.
"""
import ctypes as C
import json
import math
import os
import random
import time

import numpy as np

from . import _lib, blocks, quantize, sampling
from .blocks import (AttentionBlock, DeEmbedBlock, EmbedBlock, FastMatMulBlock, GeluBlock, LayerNormBlock,
                     ResidualBlock, SoftmaxBlock)

_FP = C.POINTER(C.c_float)
_IP = C.POINTER(C.c_int32)


_LINEAR = {"attn.c_attn.weight": (1, 3), "attn.c_proj.weight": (1, 1), "mlp.c_fc.weight": (1, 4), "mlp.c_proj.weight": (4, 1)}


def tensor_shape(name, params):
    """Shape of a tensor file of the weight directory as the forward path wants it
    (linear weights [in, out], the layout other/conversion_scripts/*.py write for HF
    GPT-2 `Conv1D` modules; model.js:404-417)."""
    d = params["n_embd"]
    if name == "transformer.wte.weight":
        return (params["vocab_size"], d)
    if name == "transformer.wpe.weight":
        return (params["n_ctx"], d)
    rest = name.split(".", 3)[3] if name.startswith("transformer.h.") else name
    if rest in _LINEAR:
        k, n = _LINEAR[rest]
        return (k * d, n * d)
    if rest.endswith(".bias") and rest[:-5] + ".weight" in _LINEAR:
        return (_LINEAR[rest[:-5] + ".weight"][1] * d,)
    return (d,)  # LayerNorm gains and biases


def read_tensor(weightsFolder, name, params):
    """One `<name>_gpt.bin` of little-endian f32 (model.js:484-488 `fetchBin`).
    Two variations of the directory that earlier versions of the reference handled
    (condensed/condensed.js:1755-1783) are accepted through params_gpt.json:
    `"bias": false` - bias files are absent and read as zeros;
    `"linear_layout": "out_in"` - the four linear weights are stored as torch
    `nn.Linear` holds them, [out, in] (nanoGPT), and are transposed here."""
    shape = tensor_shape(name, params)
    if name.endswith(".bias") and not params.get("bias", True):
        return np.zeros(shape, np.float32)
    a = np.fromfile(os.path.join(weightsFolder, name + "_gpt.bin"), dtype="<f4")
    if a.size != int(np.prod(shape)):
        raise ValueError(f"Model load failed: {name}_gpt.bin holds {a.size} values, expected {int(np.prod(shape))}.")
    if len(shape) == 2 and params.get("linear_layout", "in_out") == "out_in" and not name.startswith("transformer.w"):
        return np.ascontiguousarray(a.reshape(shape[1], shape[0]).T)
    return a.reshape(shape)


class GPT:
    def __init__(self, folder, type="bpe", tensors=None, params=None, tokenizer=None, flags=0, device_index=0, tokenization=None,
                 quantize=None):
        """`quantize="int8"` (or `"quantize": "int8"` in params_gpt.json) turns the four fp32 linear weights of
        every layer into the weight-only int8 form of other/int8-gemm.js while they are loaded
        (quantize.quantizeMatrix, per-output-column absmax); embeddings, biases and LayerNorm stay fp32."""
        self.folder = folder
        self.tokenizerType = type
        self.initialized = False
        self.device = None
        self.model = None
        self.tokenizer = tokenizer
        self.params = None
        self.externalBuffer = None
        self.unloadDeletionStack = []
        self.defaultPrompt = None
        self.defaultTopK = None
        self.defaultTemperature = None
        self.defaultTokens = None
        self._tensors = tensors
        self._params_in = params
        self._flags = flags
        self._device_index = device_index
        self._tokenization = tokenization
        if quantize not in (None, "int8"):
            raise ValueError('quantize must be None or "int8"')
        self._quantize = quantize
        self._handle = None
        self._history = []
        self.burst = 8  # tokens generate() makes per call once the window is cached (1: a call per token)
        self.lastGpuMs = 0.0

    # ---------------- lifecycle ----------------

    def initialize(self):
        if self.initialized:
            print("Model already initialized")
            return
        self.device = blocks.Device(self._device_index)  # raises if no gfx950 device: "WebGPU is not supported"
        blocks.initializeOperations(self.device)
        self.model, self.params = self.loadModel(self.folder)
        # model.js:33-34: the tokenizer of the model type, from `tokenization` (the folder the
        # reference calls weights/tokenization) unless one was handed in
        if self.tokenizer is None and self._tokenization is not None:
            from . import tokenizer as tk
            d = self._tokenization
            if self.tokenizerType == "bpe":
                tokens = os.path.join(d, "gpt_tokens.json")
                real = os.path.exists(tokens) and open(tokens, encoding="utf-8").read(64).lstrip().startswith("{")
                self.tokenizer = tk.GPT2Tokenizer().load(os.path.join(d, "vocab.bpe"), tokens if real else None)
            else:
                self.tokenizer = tk.SimpleTokenizer().load(os.path.join(d, "simple_tokens.json"))
        if self.tokenizerType == "bpe":
            self.defaultPrompt = "What is the answer to life, the universe, and everything?\n"
            self.defaultTopK, self.defaultTemperature, self.defaultTokens = 3, 1, 30
        else:
            self.defaultPrompt = "WILL:\nAh, how dare you challenge me?\nHave you forgotten I built WebGPT?\n"
            self.defaultTopK, self.defaultTemperature, self.defaultTokens = 2, 1, 80
        self.initialized = True

    def loadParameters(self, weightsFolder):
        """model.js:289-337."""
        if self._params_in is not None:
            params = dict(self._params_in)
        else:
            with open(os.path.join(weightsFolder, "params_gpt.json")) as f:
                params = json.load(f)
        if params["n_embd"] % 4 != 0:
            raise ValueError("Model load failed: n_embd must be divisible by 4.")
        if params["n_embd"] % params["n_head"] != 0:
            raise ValueError("Model load failed: n_embd must be divisible by n_head.")
        if (params["n_embd"] // params["n_head"]) % 4 != 0:
            raise ValueError("Model load failed: n_embd / n_head must be divisible by 4.")
        # The vocabulary is never split here: one buffer, one launch.
        params["vocab_chunk_size"] = params["vocab_size"]
        params["vocab_chunk_instances"] = 1
        params["head_size"] = params["n_embd"] // params["n_head"]
        params["hidden_size"] = params["n_embd"] * 4
        params["attention_scale"] = 1 / math.sqrt(params["n_embd"] / params["n_head"])
        params["bias"] = params.get("bias", True)
        return params

    def _fetch(self, weightsFolder, name, params=None):
        if self._tensors is not None:
            return self._tensors[name]
        return read_tensor(weightsFolder, name, params or self.params)

    def loadModel(self, folder):
        if self.initialized:
            print("Model already loaded")
            return None
        weightsFolder = folder
        params = self.loadParameters(weightsFolder)
        names = sorted(self._tensors) if self._tensors is not None else None
        packed = names is not None and any(n.endswith(".weight.q") for n in names)
        quantise = (self._quantize or params.get("quantize")) == "int8" and not packed
        int8 = packed or quantise
        p = _lib.Params(params["n_layer"], params["n_head"], params["n_embd"], params["n_ctx"], params["vocab_size"],
                        1 if int8 else 0, params.get("max_prefill", 0), self._flags)
        h = C.c_uint64(0)
        _lib.call("wgpt_model_create", C.byref(p), C.byref(h))
        self._handle = h.value
        if names is None:
            names = [n for n in self._directory_names(params)]
        def send(n, a):
            a = np.ascontiguousarray(a)
            _lib.call("wgpt_model_set_tensor", self._handle, n.encode(), a.ctypes.data_as(C.c_void_p), a.nbytes)

        for n in names:
            a = self._fetch(weightsFolder, n, params)
            if quantise and n.startswith("transformer.h.") and n.split(".", 3)[3] in _LINEAR:
                q, scale = quantize.quantizeMatrix(a)
                send(n + ".q", q)
                send(n + ".scale", scale)
            else:
                send(n, a)
        _lib.call("wgpt_model_finalize", self._handle)
        return {"handle": self._handle}, params

    @staticmethod
    def _directory_names(params):
        yield "transformer.wte.weight"
        yield "transformer.wpe.weight"
        for i in range(params["n_layer"]):
            for s in ("ln_1.weight", "ln_1.bias", "attn.c_attn.weight", "attn.c_attn.bias", "attn.c_proj.weight",
                      "attn.c_proj.bias", "ln_2.weight", "ln_2.bias", "mlp.c_fc.weight", "mlp.c_fc.bias",
                      "mlp.c_proj.weight", "mlp.c_proj.bias"):
                yield f"transformer.h.{i}.{s}"
        yield "transformer.ln_f.weight"
        yield "transformer.ln_f.bias"

    def unloadBuffers(self):
        for b in self.unloadDeletionStack:
            b.destroy()
        self.unloadDeletionStack = []
        if self._handle is not None:
            _lib.call("wgpt_model_destroy", self._handle)
            self._handle = None
        self.initialized = False

    def initTensor(self, data, dims, ops=("storage",)):
        buf = blocks.init_tensor(data, dims, ops)
        self.unloadDeletionStack.append(buf)
        return buf

    def bufferSize(self, dimX, dimY=1, dimZ=1):
        return dimX * dimY * dimZ * 4

    # ---------------- forward ----------------

    def prefill(self, idx):
        ids = np.ascontiguousarray(idx, dtype=np.int32)
        logits = np.empty(self.params["vocab_size"], np.float32)
        _lib.call("wgpt_prefill", self._handle, ids.ctypes.data_as(_IP), len(ids), logits.ctypes.data_as(_FP))
        self._history = [int(t) for t in ids]
        self._update_ms()
        return logits

    def decode(self, token):
        logits = np.empty(self.params["vocab_size"], np.float32)
        _lib.call("wgpt_decode", self._handle, int(token), logits.ctypes.data_as(_FP))
        self._history.append(int(token))
        self._update_ms()
        return logits

    def decode_greedy(self, token, steps, want_logits=False):
        out = np.empty(steps, np.int32)
        logits = np.empty(self.params["vocab_size"], np.float32) if want_logits else None
        _lib.call("wgpt_decode_greedy", self._handle, int(token), steps, out.ctypes.data_as(_IP),
                  logits.ctypes.data_as(_FP) if want_logits else None)
        self._history += [int(token)] + [int(t) for t in out[:-1]]
        self._update_ms()
        return (out, logits) if want_logits else out

    def decode_sample(self, token, steps, top_k, temperature, u):
        """`steps` tokens chosen on the device as GPT.generate chooses them (model.js:81-85),
        u[i] standing for the i-th Math.random() draw; the logits never leave the device."""
        u = np.ascontiguousarray(u, np.float64)
        if u.shape != (steps,):
            raise ValueError("decode_sample: one uniform draw per step")
        out = np.empty(steps, np.int32)
        _lib.call("wgpt_decode_sample", self._handle, int(token), steps, int(top_k), float(temperature),
                  u.ctypes.data_as(C.POINTER(C.c_double)), out.ctypes.data_as(_IP), None)
        self._history += [int(token)] + [int(t) for t in out[:-1]]
        self._update_ms()
        return out

    def _update_ms(self):
        ms = C.c_float(0)
        _lib.call("wgpt_model_last_gpu_ms", self._handle, C.byref(ms))
        self.lastGpuMs = ms.value

    def run(self, idx):
        """Logits of the last token of window `idx` (model.js:104). Served from the KV
        cache when `idx` extends the previous window by one token, else recomputed."""
        idx = [int(t) for t in idx]
        if self.externalBuffer is not None:
            # model.js:211-222: the residual stream after the last layer, [seq_length, n_embd], is copied into the
            # buffer a visualisation registered (visuals.js:48-50). The rows of the whole window are needed, so the
            # window is recomputed, as the reference recomputes it for every token.
            logits = self.prefill(idx)
            rows = self.tap("residual", len(idx))
            if self.bufferSize(len(idx), self.params["n_embd"]) > self.externalBuffer.size:
                raise ValueError("externalBuffer is smaller than [seq_length, n_embd]")
            self.externalBuffer.upload(rows)
            return logits
        if len(idx) == len(self._history) + 1 and len(idx) <= self.params["n_ctx"] and idx[:-1] == self._history \
                and len(self._history) > 0:
            return self.decode(idx[-1])
        return self.prefill(idx)

    def tap(self, name, rows=None):
        d = self.params["n_embd"]
        if rows is None:
            pos = C.c_int(0)
            _lib.call("wgpt_model_position", self._handle, C.byref(pos))
            rows = pos.value
        out = np.empty((rows, d), np.float32)
        _lib.call("wgpt_model_tap", self._handle, name.encode(), out.ctypes.data_as(_FP), out.size)
        return out

    def decode_bytes(self, t):
        b = C.c_uint64(0)
        _lib.call("wgpt_model_decode_bytes", self._handle, int(t), C.byref(b))
        return b.value

    def set_decode_mode(self, mode):
        _lib.call("wgpt_model_set_decode_mode", self._handle, int(mode))

    def tune_poll_delays(self, rounds=2):
        """Searches the persistent decode kernel's seven poll delays on this GPU (wgpt_model_tune_poll_delays; needs
        position 0). Returns (delays, ms_per_token_before, ms_per_token_after)."""
        chosen = (C.c_int32 * 7)()
        before, after = C.c_float(0), C.c_float(0)
        _lib.call("wgpt_model_tune_poll_delays", self._handle, int(rounds), chosen, C.byref(before), C.byref(after))
        return [int(v) for v in chosen], before.value, after.value

    def poll_delays(self):
        out = (C.c_int32 * 7)()
        _lib.call("wgpt_model_poll_delays", self._handle, out)
        return [int(v) for v in out]

    def generate(self, prompt, max_new_tokens, top_k, temperature):
        """The loop of model.js:53-102. `prompt` is a string when a tokenizer was
        given, else a list of token ids; yields decoded text or ids accordingly."""
        if not self.initialized:
            print("Model not loaded yet")
            return
        history = list(self.tokenizer.encode(prompt)) if self.tokenizer else [int(t) for t in prompt]
        warmupRuns = 3
        totalTime = 0.0
        n_ctx = self.params["n_ctx"]
        i = 0
        while i < max_new_tokens:
            idx_cond = history[-n_ctx:]
            startTime = time.perf_counter()
            h = self._history
            cached = len(h) > 0 and len(idx_cond) == len(h) + 1 and len(idx_cond) <= n_ctx and idx_cond[:-1] == h
            if cached and 1 <= top_k <= 1024 and temperature > 0:
                # the window extends the cached one by a token: that token goes in, the next one is
                # selected on the device with this draw, and the logits are never read back. Up to
                # self.burst tokens are made by one call, each with the draw the reference's loop would
                # have made for it (one per token, in order); they are yielded one by one.
                steps = max(1, min(int(self.burst), max_new_tokens - i, n_ctx - len(h)))
                draws = [random.random() for _ in range(steps)]
                ids = [int(t) for t in self.decode_sample(idx_cond[-1], steps, top_k, temperature, draws)]
                lapsed = (time.perf_counter() - startTime) * 1000.0 / steps
                for k, t in enumerate(ids):
                    if i + k >= warmupRuns:
                        totalTime += lapsed
                    history = history + [t]
                    yield self.tokenizer.decode([t]) if self.tokenizer else t
                i += steps
                continue
            logits = self.run(idx_cond)
            sel = sampling.selectTopK(logits, top_k) if top_k != 1 else \
                {"topKIndices": [int(np.argmax(logits))], "topKProbs": [float(np.max(logits))]}
            probs = sampling.cpuSoftmax(sel["topKProbs"], temperature)
            idx_next = sel["topKIndices"][sampling.sampleFromDistribution(probs)]
            lapsed = (time.perf_counter() - startTime) * 1000.0
            if i >= warmupRuns:
                totalTime += lapsed
            history = history + [idx_next]
            yield self.tokenizer.decode([idx_next]) if self.tokenizer else idx_next
            i += 1
        self.averageMs = totalTime / max(1, max_new_tokens - warmupRuns)
