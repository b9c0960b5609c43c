// Seeded synthetic tensors, bit-identical to webgpt_amd/csrc/wgpt_synth.h and
// webgpt_amd/synth.py: 32-bit integer hashing (Math.imul), exact integer sums, one
// double multiply, one rounding to float (Float32Array store).
"use strict";

function mix32(x) {
  x = x >>> 0;
  x ^= x >>> 16;
  x = Math.imul(x, 0x7feb352d) >>> 0;
  x ^= x >>> 15;
  x = Math.imul(x, 0x846ca68b) >>> 0;
  x ^= x >>> 16;
  return x >>> 0;
}

function tensorId(name) {  // FNV-1a
  let h = 2166136261;
  for (const b of Buffer.from(name, "utf8")) {
    h = Math.imul((h ^ b) >>> 0, 16777619) >>> 0;
  }
  return h >>> 0;
}

function tensorKey(seed, tid) {
  return mix32((Math.imul(seed, 0x9e3779b1) + Math.imul(tid, 0x85ebca77) + 0x165667b1) >>> 0);
}
const elemKey = (tkey, index) => mix32((tkey ^ mix32((index + 0x27d4eb2f) >>> 0)) >>> 0);
const draw = (ekey, j) => mix32((ekey + Math.imul(j, 0x9e3779b9)) >>> 0);

function normal(seed, name, count, std = 0.02) {
  const key = tensorKey(seed, tensorId(name));
  const out = new Float32Array(count);
  const scale = std / 16777216.0;
  for (let i = 0; i < count; i++) {
    const e = elemKey(key, i);
    let sum = 0;
    for (let j = 0; j < 12; j++) sum += draw(e, j) >>> 8;
    out[i] = (sum - 6 * 16777216) * scale;
  }
  return out;
}

function tokens(seed, name, count, vocab) {
  const key = tensorKey(seed, tensorId(name));
  const out = new Int32Array(count);
  for (let i = 0; i < count; i++) out[i] = draw(elemKey(key, i), 0) % vocab;
  return out;
}

function int8Packed(seed, name, K, N) {
  const key = tensorKey(seed, tensorId(name));
  const out = new Int32Array(K * (N / 4));
  for (let w = 0; w < out.length; w++) {
    let word = 0;
    for (let e = 0; e < 4; e++) {
      const q = (draw(elemKey(key, w * 4 + e), 0) % 255) - 127;
      word |= (q & 0xff) << (8 * e);
    }
    out[w] = word;
  }
  return out;
}

function uniform(seed, name, count, lo, hi) {
  const key = tensorKey(seed, tensorId(name));
  const out = new Float32Array(count);
  const step = (hi - lo) / 16777216.0;
  for (let i = 0; i < count; i++) out[i] = lo + (draw(elemKey(key, i), 0) >>> 8) * step;
  return out;
}

const CONFIGS = {
  "toy": { n_layer: 6, n_head: 6, n_embd: 384, n_ctx: 256, vocab_size: 65, prompt: 64, decode: 128, dtype: "f32" },
  "gpt2-117m": { n_layer: 12, n_head: 12, n_embd: 768, n_ctx: 1024, vocab_size: 50257, prompt: 128, decode: 256, dtype: "f32" },
  "gpt2-345m": { n_layer: 24, n_head: 16, n_embd: 1024, n_ctx: 1024, vocab_size: 50257, prompt: 512, decode: 512, dtype: "f32" },
  "gpt2-774m": { n_layer: 36, n_head: 20, n_embd: 1280, n_ctx: 1024, vocab_size: 50257, prompt: 64, decode: 960, dtype: "f32" },
  "gpt2-1.5b": { n_layer: 48, n_head: 25, n_embd: 1600, n_ctx: 1024, vocab_size: 50257, prompt: 128, decode: 256, dtype: "f32" },
  "gpt2-1.5b-int8": { n_layer: 48, n_head: 25, n_embd: 1600, n_ctx: 1024, vocab_size: 50257, prompt: 128, decode: 256, dtype: "int8" },
};

// Yields [name, TypedArray] for the whole weight directory of a configuration.
function* makeTensors(cfg, seed, fast) {
  const d = cfg.n_embd, V = cfg.vocab_size;
  const gen = (name, count) => (fast ? fast(seed, name, count, 0.02) : normal(seed, name, count));
  const ones = (n) => new Float32Array(n).fill(1);
  const lin = function* (name, K, N) {
    if (cfg.dtype === "int8") {
      yield [name + ".q", int8Packed(seed, name + ".q", K, N)];
      yield [name + ".scale", uniform(seed, name + ".scale", N, 1e-3, 1e-2)];
    } else {
      yield [name, gen(name, K * N)];
    }
  };
  yield ["transformer.wte.weight", gen("transformer.wte.weight", V * d)];
  yield ["transformer.wpe.weight", gen("transformer.wpe.weight", cfg.n_ctx * d)];
  for (let i = 0; i < cfg.n_layer; i++) {
    const p = `transformer.h.${i}.`;
    yield [p + "ln_1.weight", ones(d)];
    yield [p + "ln_1.bias", new Float32Array(d)];
    yield* lin(p + "attn.c_attn.weight", d, 3 * d);
    yield [p + "attn.c_attn.bias", gen(p + "attn.c_attn.bias", 3 * d)];
    yield* lin(p + "attn.c_proj.weight", d, d);
    yield [p + "attn.c_proj.bias", gen(p + "attn.c_proj.bias", d)];
    yield [p + "ln_2.weight", ones(d)];
    yield [p + "ln_2.bias", new Float32Array(d)];
    yield* lin(p + "mlp.c_fc.weight", d, 4 * d);
    yield [p + "mlp.c_fc.bias", gen(p + "mlp.c_fc.bias", 4 * d)];
    yield* lin(p + "mlp.c_proj.weight", 4 * d, d);
    yield [p + "mlp.c_proj.bias", gen(p + "mlp.c_proj.bias", d)];
  }
  yield ["transformer.ln_f.weight", ones(d)];
  yield ["transformer.ln_f.bias", new Float32Array(d)];
}

module.exports = { mix32, tensorId, normal, tokens, int8Packed, uniform, CONFIGS, makeTensors };
