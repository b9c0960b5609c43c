// Runs the toy GPT through the JavaScript host on the GPU and prints results as JSON:
// run() over a growing window (prefill once, then KV-cached decodes), the block-by-block
// replay of the reference's pass list, generate() with top_k = 1 and the on-device greedy loop.
"use strict";
const w = require("../../webgpt_amd/js/index.js");
const s = w.synth;

async function main() {
  const name = process.argv[2] || "toy";
  const cfg = s.CONFIGS[name];
  const fast = (seed, n, count, std) => w.native.synthNormal(seed, n, count, std);
  const tensors = {};
  for (const [n, a] of s.makeTensors(cfg, 1, fast)) tensors[n] = a;
  const params = { n_layer: cfg.n_layer, n_head: cfg.n_head, n_embd: cfg.n_embd, n_ctx: cfg.n_ctx, vocab_size: cfg.vocab_size };
  const gpt = new w.GPT(null, "char", { tensors, params });
  await gpt.initialize();
  const tokens = Array.from(s.tokens(1, "prompt", 24, cfg.vocab_size));
  const out = { device: gpt.device.name, tokens };
  let logits = await gpt.run(tokens.slice(0, 16));
  out.logits16 = Array.from(logits);
  for (let t = 16; t < 24; t++) logits = await gpt.run(tokens.slice(0, t + 1));
  out.logits24 = Array.from(logits);
  // the reference's pass list, block by block, whole window recomputed
  const bw = gpt.loadBlockWeights(tensors);
  out.blocks24 = Array.from(await gpt.runBlocks(tokens, bw));
  // the same pass list over the table held as the reference holds it: zero-padded [chunk, d] gather chunks and
  // host-transposed [d, chunk] de-embedding chunks (model.js:298-364), here two chunks of 36 rows for 65
  {
    const { n_embd: d, vocab_size: V } = gpt.params;
    const chunk = 36, padded = new Float32Array(2 * chunk * d);
    padded.set(tensors["transformer.wte.weight"]);
    const gather = [0, 1].map((i) => w.initTensor(padded.subarray(i * chunk * d, (i + 1) * chunk * d), [chunk, d]));
    const transposed = [0, 1].map((i) => w.initTensor(Float32Array.from(w.transpose(padded.subarray(i * chunk * d, (i + 1) * chunk * d), chunk, d)), [d, chunk]));
    out.chunked24 = Array.from(await gpt.runBlocks(tokens, bw, { vocab_chunk_size: chunk, embdBuffers: gather, deEmbeddingsBuffers: transposed }));
    gather.concat(transposed).forEach((b) => b.destroy());
    // softmax with the transposed store (instructions.js:594)
    const sm = w.initTensor(new Float32Array([0, 1, 2, 3, 1, 1]), [2, 3]);
    const inst = w.SoftmaxBlock.newInstance(2, 3, sm, true);
    w.runPasses(inst.passes);
    out.softmaxT = Array.from(inst.resultBuffer.download());
    sm.destroy();
    w.clearOperationCache();
  }
  // GPT.externalBuffer (model.js:211-222, visuals.js:48-50): run() leaves the last layer's residual rows there
  {
    const ext = new w.DeviceBuffer([cfg.n_ctx, cfg.n_embd]);
    gpt.externalBuffer = ext;
    out.extLogits = Array.from(await gpt.run(tokens.slice(0, 20)));
    out.extRows = Array.from(ext.download(0, 4 * 20 * cfg.n_embd));
    gpt.externalBuffer = undefined;
    ext.destroy();
  }
  // error path: the library's message becomes a thrown Error
  try { await gpt.run([cfg.vocab_size]); out.badToken = null; } catch (e) { out.badToken = e.message; }
  // generate() with top_k = 1, then the same continuation on the device
  const gen = [];
  for await (const id of gpt.generate(tokens.slice(0, 8), 10, 1, 1.0)) gen.push(id);
  out.generated = gen;
  const lg = await gpt.run(tokens.slice(0, 8));
  let first = 0;
  for (let i = 1; i < lg.length; i++) if (lg[i] > lg[first]) first = i;
  out.greedy = [first].concat(Array.from(gpt.decodeGreedy(first, 9)));
  // generate() with top_k = 3 and a seeded Math.random: a call per token, bursts of 8, bursts of 5 (19 tokens: no
  // multiple of either)
  {
    const realRandom = Math.random;
    out.bursts = {};
    for (const burst of [1, 8, 5]) {
      let state = 12345;
      Math.random = () => { state = (state * 1103515245 + 12345) % 2147483648; return state / 2147483648; };
      gpt.burst = burst;
      gpt._history = [];
      const ids = [];
      for await (const id of gpt.generate(tokens.slice(0, 8), 19, 3, 0.9)) ids.push(id);
      out.bursts[burst] = ids;
    }
    Math.random = realRandom;
    gpt.burst = 8;
  }
  // token selection on the device: one buffer-level call, then a sampled continuation
  const probe = new Float32Array([0.5, 2.0, -1.0, 2.0, 1.5]);
  const pb = w.initTensor(probe, [5]);
  const sel = w.native.sampleTopK(5, 3, 0.5, 0.6, pb.handle);
  out.select = { id: sel.id, topKIndices: Array.from(sel.topKIndices), probs: Array.from(sel.probs) };
  pb.destroy();
  await gpt.run(tokens.slice(0, 8));
  out.draws = [0.05, 0.5, 0.95, 0.3];
  out.sampled = Array.from(gpt.decodeSample(first, 4, 0.9, out.draws));
  gpt.unloadBuffers();
  w.destroyOperations();
  console.log(JSON.stringify(out));
}
main().catch((e) => { console.error(e); process.exit(1); });
