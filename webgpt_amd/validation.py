"""The validation harness of other/validation/validation.js: a JSON array with one entry per
generation step, each mapping a tap name (tok_pos_emb, block<i>_{ln1,attn,r1,ln2,mlp,r2}, ln_f,
logits; validation.js:113-134) to {"shape": [1, T, n], "data": nested lists}, produced by a
reference model generating greedily (top_k = 1) and compared with this model step by step.

`dump` writes that schema from a loaded GPT, `validate` consumes it. The GPT must have been
created with flags=FLAG_TAPS so that the activations of a window stay readable."""
import json

import numpy as np

from . import _lib


def tap_names(n_layer):
    names = ["tok_pos_emb"]
    for i in range(n_layer):
        names += [f"block{i}_{s}" for s in ("ln1", "attn", "r1", "ln2", "mlp", "r2")]
    return names + ["ln_f"]


def load(path_or_list):
    """loadValidateModel (validation.js:183-205): values parsed as floats into Float32 arrays
    of the stated shape."""
    steps = path_or_list
    if isinstance(path_or_list, str):
        with open(path_or_list) as f:
            steps = json.load(f)
    out = []
    for step in steps:
        loaded = {}
        for key, entry in step.items():
            shape = tuple(int(s) for s in entry["shape"])
            data = np.array(entry["data"], dtype=np.float64).astype(np.float32)
            if data.size != int(np.prod(shape)):
                raise ValueError(f"validation entry {key}: {data.size} values for shape {list(shape)}")
            loaded[key] = data.reshape(shape)
        out.append(loaded)
    return out


def _entry(a):
    a = np.asarray(a, np.float32)
    a3 = a.reshape((1,) + a.shape) if a.ndim == 2 else a.reshape(1, 1, -1)
    return {"shape": list(a3.shape), "data": a3.tolist()}


def dump(gpt, prompt, steps, path=None):
    """Greedy generation of `steps` tokens from `prompt` (token ids), one whole-window forward
    per step as the reference runs, every tap recorded. Returns the list; writes JSON to path."""
    history = [int(t) for t in prompt]
    out = []
    n_layer = gpt.params["n_layer"]
    for _ in range(steps):
        window = history[-gpt.params["n_ctx"]:]
        logits = gpt.prefill(window)
        step = {name: _entry(gpt.tap(name, len(window))) for name in tap_names(n_layer)}
        step["logits"] = _entry(logits)
        out.append(step)
        history.append(int(np.argmax(logits)))   # top_k = 1: lowest index on ties, as np.argmax
    if path is not None:
        with open(path, "w") as f:
            json.dump(out, f)
    return out


def validate(gpt, steps, prompt, tolerance=1e-3):
    """runGPTValidation (validation.js:30-137): for every step runs the window, compares every
    recorded tap and the logits, and feeds back the arg-max. The reference's check is
    `a - b > 0.001` per element (validation.js:207-222); here the absolute difference is used.
    Returns a list of (step, key, worst absolute difference) for the entries that fail."""
    steps = load(steps)
    history = [int(t) for t in prompt]
    failures = []
    for si, want in enumerate(steps):
        window = history[-gpt.params["n_ctx"]:]
        logits = gpt.prefill(window)
        for key, ref in want.items():
            if key == "logits":
                got = logits
                ref = ref.reshape(-1, ref.shape[-1])[-1]      # the last position's row
            else:
                got = gpt.tap(key, len(window))
                ref = ref.reshape(got.shape)
            worst = float(np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64))))
            if not worst <= tolerance:
                failures.append((si, key, worst))
        history.append(int(np.argmax(logits)))
    return failures
