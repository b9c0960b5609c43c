// Prints, as JSON, values computed by the JavaScript host without a GPU.
"use strict";
const w = require("../../webgpt_amd/js/index.js");
const s = w.synth;
const out = {
  exports: w.native.exports(),
  names: Object.keys(w).sort(),
  normal: Array.from(s.normal(7, "transformer.h.3.mlp.c_fc.bias", 64)),
  tokens: Array.from(s.tokens(3, "prompt", 64, 50257)),
  int8: Array.from(s.int8Packed(3, "x.q", 8, 16)),
  uniform: Array.from(s.uniform(3, "s", 33, 1e-3, 1e-2)),
  nativeNormal: Array.from(w.native.synthNormal(7, "transformer.h.3.mlp.c_fc.bias", 64, 0.02)),
  tensorId: s.tensorId("transformer.wte.weight"),
  topk: w.selectTopK(new Float32Array([0.5, 2.0, -1.0, 2.0, 1.5]), 3),
  top1: w.selectTopK(new Float32Array([0.5, 2.0, -1.0, 2.0, 1.5]), 1),
  softmax: w.cpuSoftmax([1.0, 2.0, 4.0], 0.5),
  sample: [0.0, 0.19, 0.2, 0.49, 0.5, 0.999].map((r) => w.sampleFromDistribution([0.2, 0.3, 0.5], r)),
  transpose: Array.from(w.transpose(new Float32Array([1, 2, 3, 4, 5, 6]), 2, 3)),
  wgSize: [w.wgSize(65, 32), w.wgSize(64, 32)],
  errors: {},
  gptMethods: Object.getOwnPropertyNames(w.GPT.prototype).sort(),
};
// quantizeMatrix / dequantizeMatrix (other/int8-gemm.js:25-62) on a seeded matrix and on the rounding probes
{
  const K = 24, N = 8;
  const m = s.normal(9, "quantize.probe", K * N);
  m[5] = 0; m[N + 2] = -m[2];
  for (let k = 0; k < K; k++) m[k * N + 7] = 0;  // an all-zero column
  const q = w.quantizeMatrix(m, K, N);
  out.quant = { words: Array.from(q.quantizedMatrix), scale: Array.from(q.scale), dequant: Array.from(w.dequantizeMatrix(q.quantizedMatrix, q.scale, K, N)) };
  const probe = new Float32Array([-0.5 / 127, 0.5 / 127, -1.5 / 127, 1.0, 2.5 / 127, -2.5 / 127, -1.0, 0.0]);
  out.quantProbe = Array.from(w.quantizeMatrix(probe, 1, 8, 1.0).quantizedMatrix);
}
const dev = { limits: { maxStorageBufferBindingSize: 1 << 20 } };
w.initializeOperations(dev);
const tryErr = (name, f) => { try { f(); out.errors[name] = null; } catch (e) { out.errors[name] = e.message; } };
const fake = { handle: 1, dims: [1] };
tryErr("matmul", () => w.FastMatMulBlock.newInstance(1, 12, 4, fake, fake, fake));
tryErr("residual", () => w.ResidualBlock.newInstance(1, 6, fake, fake));
tryErr("layernorm", () => w.LayerNormBlock.newInstance(1, 6, fake, fake, fake));
tryErr("gelu", () => w.GeluBlock.newInstance(1, 6, fake));
tryErr("bufferSize", () => w.FastMatMulBlock.bufferSize(1 << 20, 1));
tryErr("device", () => new w.Device(0));
console.log(JSON.stringify(out));
