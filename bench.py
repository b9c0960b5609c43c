#!/usr/bin/env python3
"""Benchmark of the per-token forward path: GPT-2 117M fp32 batch-1 greedy decode.

One "step" is one decode token: the whole forward of one new token against the
device-resident KV cache, followed by the on-device arg-max that feeds the next
step. Weights, KV cache and the first token are resident in HBM when the timed
region starts; nothing crosses PCIe inside it. Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config gpt2-117m] [--prompt T]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E
MFMA_FP32_PEAK_FLOPS = 157.3e12  # MI355X dense fp32 matrix


def probe_webgpu_adapter():
    """Looks for what the reference itself would need to run on the host cores: node with a WebGPU binding
    (the `webgpu` / `dawn.node` modules) or a Chromium that accepts --use-webgpu-adapter=swiftshader. Returns a
    short description of what was found; nothing is installed or downloaded."""
    import shutil
    import subprocess
    found = []
    node = shutil.which("node")
    if node:
        for mod in ("webgpu", "dawn.node", "@webgpu/dawn"):
            try:
                r = subprocess.run([node, "-e", f"const m = require('{mod}'); process.exit(m ? 0 : 1)"],
                                   capture_output=True, timeout=20)
                if r.returncode == 0:
                    found.append(f"node module {mod}")
            except (OSError, subprocess.SubprocessError):
                pass
        try:
            r = subprocess.run([node, "-e", "process.exit(typeof navigator !== 'undefined' && navigator.gpu ? 0 : 1)"],
                               capture_output=True, timeout=20)
            if r.returncode == 0:
                found.append("navigator.gpu in node")
        except (OSError, subprocess.SubprocessError):
            pass
    browsers = [b for b in ("chromium", "chromium-browser", "google-chrome", "chrome") if shutil.which(b)]
    if found:
        return "found, not used: " + ", ".join(found)
    return ("none found (probed: node " + ("present" if node else "absent") + ", modules webgpu / dawn.node / @webgpu/dawn, "
            "navigator.gpu, browsers " + (", ".join(browsers) if browsers else "none") + ")")


def cpu_baseline(cfg, tensors, prompt, budget_s=20.0):
    """The CPU restatement of the reference's kernels (oracle/), run the way the
    reference runs: every token recomputes the whole window (model.js:69,104)."""
    from oracle import ref
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from helpers import oracle_weights
    from webgpt_amd import synth
    w, p = oracle_weights(tensors, cfg), synth.model_params(cfg)
    hist = [int(t) for t in prompt]
    times = []
    t_all = time.perf_counter()
    while len(times) < 8 and (time.perf_counter() - t_all) < budget_s:
        t0 = time.perf_counter()
        logits = ref.forward(p, w, np.array(hist, np.int32))
        times.append(time.perf_counter() - t0)
        hist.append(int(np.argmax(logits)))
    ms = 1000.0 * float(np.mean(times))
    # The reference on a CPU WebGPU adapter (Dawn/SwiftShader) is the baseline the configuration names; it is
    # reported instead of this port only if such an adapter exists on the machine, and the line says which it was.
    return {"value": round(ms, 3), "unit": "ms/token", "cores": ref.get_threads(), "kind": "port",
            "adapter": probe_webgpu_adapter(),
            "sample": f"{len(times)} greedy tokens after a {len(prompt)}-token prompt, whole window recomputed per "
                      f"token as GPT.run does, C restatement of the WGSL kernels with OpenMP"}


# HBM bytes of one decode step, from rocprofv3 --pmc counter runs (FETCH_SIZE x the copy-probe factor + WRITE_SIZE)
# on single-token launches of the persistent kernel: bytes, the contexts of the profiled launches, the profile that
# holds the figures and the first 16 hex digits of the SHA-256 of the kernel's source file when it was profiled.
MEASURED_TRAFFIC = {
    "gpt2-117m": (515.8e6, (133, 164), "profiles/decode_persistent_gpt2-117m.md", "7b7ce1999a5b27ff"),
    "gpt2-345m": (1557.9e6, (555, 586), "profiles/decode_persistent_other_configs.md", "7b7ce1999a5b27ff"),
    "gpt2-774m": (3178.0e6, (107, 138), "profiles/decode_persistent_other_configs.md", "7b7ce1999a5b27ff"),
    "gpt2-1.5b-int8": (2116.9e6, (171, 202), "profiles/decode_persistent_other_configs.md", "7b7ce1999a5b27ff"),
}
KERNEL_SOURCE = os.path.join(ROOT, "webgpt_amd", "csrc", "decode_persistent.hip")


def measured_traffic(config, persistent, ctx_lo, ctx_hi):
    """(bytes or None, where the figure comes from). A counter figure is reported only for the kernel it was
    measured on (same source file) and for a run whose contexts overlap the profiled ones; otherwise the line
    says why there is none, so a stale figure cannot pass for a measurement of this run."""
    import hashlib
    if not persistent or config not in MEASURED_TRAFFIC:
        return None, "no counter run for this configuration and decode path"
    nbytes, (lo, hi), profile, sha = MEASURED_TRAFFIC[config]
    try:
        now = hashlib.sha256(open(KERNEL_SOURCE, "rb").read()).hexdigest()[:16]
    except OSError:
        now = "source not found"
    where = {"profile": profile, "contexts": [lo, hi], "kernel_source_sha256_16": sha}
    if now != sha:
        where["stale"] = f"kernel source is now {now}: counters not re-collected since it changed"
        return None, where
    if ctx_hi < lo or ctx_lo > hi:
        where["skipped"] = f"this run's contexts {ctx_lo}..{ctx_hi} do not overlap the profiled ones"
        return None, where
    return nbytes, where


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed decode steps (default: the configuration's decode length minus the warm-up steps)")
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="gpt2-117m")
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=None,
                    help="prompt length (default: the configuration's); the decode steps that follow must fit n_ctx")
    ap.add_argument("--mode", type=int, default=None, help="decode implementation (default: library default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--tune-delays", type=int, default=0, metavar="ROUNDS",
                    help="before anything is timed, search the persistent kernel's poll delays on this GPU "
                         "(wgpt_model_tune_poll_delays) with this many passes")
    ap.add_argument("--copy-probe", action="store_true",
                    help="first run three 256 MiB device-to-device copies (a kernel of known traffic, for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (batch-1 decode does not shard usefully); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)

    from webgpt_amd import synth
    from webgpt_amd.model import GPT
    from webgpt_amd._lib import WgptError

    cfg = dict(synth.CONFIGS[args.config])
    if args.prompt is not None:
        cfg["prompt"] = args.prompt
    if args.steps is None:
        args.steps = min(cfg["decode"], cfg["n_ctx"] - cfg["prompt"]) - args.warmup
    if args.steps < 1 or cfg["prompt"] + args.warmup + args.steps > cfg["n_ctx"]:
        print(f"bench.py: prompt {cfg['prompt']} + warmup + steps exceeds n_ctx {cfg['n_ctx']}", file=sys.stderr)
        sys.exit(2)
    if args.copy_probe:
        from webgpt_amd import _lib, blocks
        blocks.Device(0)
        n = 256 << 20
        src, dst = blocks.Buffer([n // 4]), blocks.Buffer([n // 4])
        for _ in range(3):
            _lib.call("wgpt_copy", dst.handle, 0, src.handle, 0, n)
        _lib.call("wgpt_sync")
        src.destroy()
        dst.destroy()
    tensors = dict(synth.make_tensors(cfg, args.seed))
    prompt = synth.make_prompt(cfg, args.seed)
    gpt = GPT(None, "bpe", tensors=tensors, params=synth.model_params(cfg))
    gpt.initialize()
    if args.mode is not None:
        gpt.set_decode_mode(args.mode)
    tuned = None
    if args.tune_delays > 0 and args.mode in (None, 1):
        try:
            t0 = time.perf_counter()
            row, before, after = gpt.tune_poll_delays(args.tune_delays)
            tuned = {"delays": row, "ms_per_token_before": round(before, 5), "ms_per_token_after": round(after, 5),
                     "search_s": round(time.perf_counter() - t0, 2)}
        except WgptError as e:
            tuned = {"error": str(e)}

    # prefill (untimed for the headline; reported separately)
    gpt.prefill(prompt)  # first call also loads the code objects
    runs = []
    for _ in range(5):
        t0 = time.perf_counter()
        logits = gpt.prefill(prompt)
        runs.append(((time.perf_counter() - t0) * 1000.0, gpt.lastGpuMs))
    prefill_wall_ms, prefill_gpu_ms = float(np.median([r[0] for r in runs])), float(np.median([r[1] for r in runs]))
    tok = int(np.argmax(logits))
    T, L, d = len(prompt), cfg["n_layer"], cfg["n_embd"]
    prefill_flops = 2.0 * T * 12 * L * d * d + 2.0 * L * T * T * d

    # warmup steps, then exactly K timed steps, all on the device
    pos = len(prompt)
    if args.warmup > 0:
        ids = gpt.decode_greedy(tok, args.warmup)
        tok = int(ids[-1])
        pos += args.warmup
    gpt.device.sync()
    t0 = time.perf_counter()
    ids = gpt.decode_greedy(tok, args.steps)
    gpt.device.sync()
    wall_ms = (time.perf_counter() - t0) * 1000.0
    gpu_ms = gpt.lastGpuMs
    ms_per_step = wall_ms / args.steps
    bytes_total = sum(gpt.decode_bytes(pos + i) for i in range(args.steps))
    achieved = bytes_total / (gpu_ms * 1e-3) / 1e9

    # per-token host loop with logits read-back (what GPT.run returns), PCIe inclusive
    per_tok = []
    nxt = int(ids[-1])
    for _ in range(min(32, cfg["n_ctx"] - pos - args.steps)):
        t0 = time.perf_counter()
        lg = gpt.decode(nxt)
        per_tok.append((time.perf_counter() - t0) * 1000.0)
        nxt = int(np.argmax(lg))

    # GPT.generate as a caller uses it (model.js:53-102): the prompt's window once, then tokens in bursts of gpt.burst
    # per call, selected on the device; its own averageMs (wall clock per token after three warm-up tokens)
    gen = None
    n_gen = min(67, cfg["n_ctx"] - len(prompt))
    if n_gen > 8:
        for _ in gpt.generate([int(t) for t in prompt], n_gen, 1, 1.0):
            pass
        gen = {"value": round(gpt.averageMs, 4), "tokens": n_gen, "burst": gpt.burst, "top_k": 1,
               "note": "GPT.generate() per token, wall clock, ids to the host; the window is cached on the device"}

    persistent = args.mode == 1
    if args.mode is None:
        try:  # the default mode is the persistent kernel wherever the library offers it for the shape
            gpt.set_decode_mode(1)
            persistent = True
        except WgptError:
            persistent = False
    kernel_name = ("decode_persistent_kernel (one launch runs all timed steps; one step = one token)" if persistent
                   else "per-block kernels (all launches of one token)")
    traffic, traffic_from = measured_traffic(args.config, persistent, pos, pos + args.steps - 1)
    out = {
        "metric": "ms/token + achieved HBM GB/s, GPT-2 117M fp32 batch-1 decode" if args.config == "gpt2-117m"
                  else f"ms/token + achieved HBM GB/s, {args.config} batch-1 decode",
        "value": round(ms_per_step, 5),
        "unit": "ms/token",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if cfg["dtype"] == "f32" else "f32 activations, int8 weights",
        "data": "synthetic",
        "config": {"workload": f"{args.config}: L{cfg['n_layer']} H{cfg['n_head']} d{cfg['n_embd']} V{cfg['vocab_size']}, "
                               f"prompt {cfg['prompt']}, greedy decode, context {pos}..{pos + args.steps - 1}",
                   "seed": args.seed},
        "tokens_per_s": round(1000.0 / ms_per_step, 1),
        "gpu_ms_per_token": round(gpu_ms / args.steps, 5),
        "prefill_tokens_per_s": round(len(prompt) / (prefill_gpu_ms * 1e-3), 1),
        "prefill_ms": round(prefill_gpu_ms, 3),  # HIP-event time, median of 5 calls after one untimed
        "prefill_wall_ms": round(prefill_wall_ms, 3),
        # whole prefill (all kernels) against the fp32 MFMA peak: linear-layer flops 2*T*12*L*d^2 + causal attention 2*L*T^2*d
        "prefill_tflops": round(prefill_flops / (prefill_gpu_ms * 1e-3) / 1e12, 2),
        "prefill_frac_of_fp32_mfma_peak": round(prefill_flops / (prefill_gpu_ms * 1e-3) / MFMA_FP32_PEAK_FLOPS, 4),
        "host_loop_ms_per_token": {"mean": round(float(np.mean(per_tok)), 4), "p50": round(float(np.median(per_tok)), 4),
                                   "note": "wgpt_decode per token incl. the logits handed to the host over PCIe"} if per_tok else None,
        "generate_ms_per_token": gen,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic, "traffic_from": traffic_from,
                     "kernel": kernel_name,
                     "bytes_per_step": int(bytes_total / args.steps),
                     "note": "achieved = algorithmic bytes (weights + KV rows read) of the timed steps / HIP-event time of "
                             "the launch(es) that ran them; traffic = measured HBM bytes of one step (rocprofv3 FETCH_SIZE + "
                             "WRITE_SIZE, profiles/) as counted on single-step launches (a launch of several steps keeps "
                             "up to a third of the vocabulary table in LDS and registers and reads that much less per step), "
                             "null where no counter run exists for the configuration"},
    }
    if persistent:
        try:
            out["poll_delays"] = {"in_use": gpt.poll_delays(), "tuned_on_this_gpu": tuned}
        except WgptError:
            pass
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, tensors, prompt)
    gpt.unloadBuffers()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
