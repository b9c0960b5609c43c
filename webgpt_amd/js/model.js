// GPT: the driver class of the reference's model.js over the HIP library.
//
// initialize() loads a weight directory (params_gpt.json + one little-endian f32
// <tensor>_gpt.bin per tensor, model.js:270-488) or takes tensors from memory;
// run(idx) resolves to the logits of the last token of the window idx
// (model.js:104-268); generate() is the sampling loop of model.js:53-102.
// run() is served from the device-resident KV cache whenever idx is the previous
// window plus one token, else the whole window is recomputed (as the reference does
// every token). runBlocks(idx) replays the reference's pass list block by block.
"use strict";
const fs = require("fs");
const path = require("path");
const { performance } = require("perf_hooks");
const native = require("./native.js");
const { Device, initTensor, runPasses } = require("./instructions.js");
const G = require("./globals.js");
const { GPT2Tokenizer, SimpleTokenizer } = require("./tokenizer.js");
const { quantizeMatrix } = require("./quantize.js");

class GPT {
  constructor(folder, type, options = {}) {
    this.folder = folder;
    this.tokenizerType = type;
    this.initialized = false;
    this.device = undefined;
    this.model = undefined;
    this.tokenizer = options.tokenizer;
    this.params = undefined;
    this.minBufferOffset = 1;
    this.defaultPrompt = undefined;
    this.defaultTopK = undefined;
    this.defaultTemperature = undefined;
    this.defaultTokens = undefined;
    this.externalBuffer = undefined;
    this.unloadDeletionStack = [];
    this._tensors = options.tensors;  // Map or object name -> TypedArray, instead of files
    this._paramsIn = options.params;
    this._flags = options.flags || 0;
    this._tokenization = options.tokenization;
    this._quantize = options.quantize;  // "int8": quantise the fp32 linear weights while loading (quantize.js)
    this._history = [];
    this.lastGpuMs = 0;
    this.burst = options.burst || 8;  // tokens generate() makes per call once the window is cached (1: a call per token)
  }

  async initialize() {
    if (this.initialized) return console.error("Model already initialized");
    this.device = new Device(0);
    G.initializeOperations(this.device);
    [this.model, this.params] = await this.loadModel(this.folder);
    // model.js:33-34: the tokenizer of the model type, from options.tokenization (the folder
    // the reference calls weights/tokenization) unless one was handed in
    if (!this.tokenizer && this._tokenization) {
      const dir = this._tokenization;
      if (this.tokenizerType == "bpe") {
        const tokens = path.join(dir, "gpt_tokens.json");
        const real = fs.existsSync(tokens) && fs.readFileSync(tokens, "utf8").trimStart().startsWith("{");
        this.tokenizer = await new GPT2Tokenizer().load(path.join(dir, "vocab.bpe"), real ? tokens : undefined);
      } else {
        this.tokenizer = await new SimpleTokenizer().load(path.join(dir, "simple_tokens.json"));
      }
    }
    if (this.tokenizerType == "bpe") {
      this.defaultPrompt = `What is the answer to life, the universe, and everything?\n`;
      this.defaultTopK = 3;
      this.defaultTemperature = 1;
      this.defaultTokens = 30;
    } else {
      this.defaultPrompt = `WILL:\nAh, how dare you challenge me?\nHave you forgotten I built WebGPT?\n`;
      this.defaultTopK = 2;
      this.defaultTemperature = 1;
      this.defaultTokens = 80;
    }
    this.initialized = true;
  }

  async *generate(prompt, max_new_tokens, top_k, temperature) {
    if (!this.initialized) {
      console.error("Model not loaded yet");
      return;
    }
    // prompt: a string when a tokenizer was given, else an array of token ids
    let history = this.tokenizer ? this.tokenizer.encode(prompt) : Array.from(prompt);
    const warmupRuns = 3;
    let totalTime = 0;
    for (let i = 0; i < max_new_tokens; i++) {
      const idx_cond = history.slice(-this.params.n_ctx);
      const startTime = performance.now();
      let idx_next;
      const h = this._history;
      const cached = h.length > 0 && idx_cond.length === h.length + 1 && idx_cond.length <= this.params.n_ctx && h.every((t, j) => t === idx_cond[j]);
      if (cached && top_k >= 1 && top_k <= 1024 && temperature > 0) {
        // the window extends the cached one by a token: that token goes in, the next one is selected
        // on the device (selectTopK, cpuSoftmax, sampleFromDistribution with this Math.random() draw)
        // and the logits are never read back. Up to `burst` tokens are made by one call, each with the
        // draw the reference's loop would have made for it (one Math.random() per token, in order); they
        // are yielded one by one. burst = 1 is a call per token.
        const room = this.params.n_ctx - h.length;  // positions the cache still has
        const steps = Math.max(1, Math.min(this.burst | 0, max_new_tokens - i, room));
        const draws = [];
        for (let k = 0; k < steps; k++) draws.push(Math.random());
        const ids = this.decodeSample(idx_cond[idx_cond.length - 1], top_k, temperature, draws);
        const lapsed = (performance.now() - startTime) / steps;
        for (let k = 0; k < steps; k++) {
          i + k >= warmupRuns && (totalTime += lapsed);
          history = history.concat(ids[k]);
          yield this.tokenizer ? this.tokenizer.decode([ids[k]]) : ids[k];
        }
        i += steps - 1;
        continue;
      } else {
        const logits = await this.run(idx_cond);
        const { topKIndices, topKProbs } = G.selectTopK(logits, top_k);
        const probs = G.cpuSoftmax(topKProbs, temperature);
        idx_next = topKIndices[G.sampleFromDistribution(probs)];
      }
      const lapsedTime = performance.now() - startTime;
      i >= warmupRuns && (totalTime += lapsedTime);
      history = history.concat(idx_next);
      yield this.tokenizer ? this.tokenizer.decode([idx_next]) : idx_next;
    }
    this.averageMs = totalTime / Math.max(1, max_new_tokens - warmupRuns);
  }

  async run(idx) {
    if (this.externalBuffer) {
      // model.js:211-222: the residual stream after the last layer, [seq_length, n_embd], is copied into the buffer a
      // visualisation registered (visuals.js:48-50). The rows of the whole window are needed, so the window is
      // recomputed, as the reference recomputes it for every token.
      const lg = native.prefill(this.model.handle, Int32Array.from(idx), this.params.vocab_size);
      this._history = Array.from(idx);
      this.lastGpuMs = native.modelLastGpuMs(this.model.handle);
      if (this.bufferSize(idx.length, this.params.n_embd) > this.externalBuffer.size) throw new Error("externalBuffer is smaller than [seq_length, n_embd]");
      this.externalBuffer.upload(native.modelTap(this.model.handle, "residual", idx.length * this.params.n_embd));
      return lg;
    }
    const h = this._history;
    const extends1 = h.length > 0 && idx.length === h.length + 1 && idx.length <= this.params.n_ctx && h.every((t, i) => t === idx[i]);
    let logits;
    if (extends1) {
      logits = native.decode(this.model.handle, idx[idx.length - 1], this.params.vocab_size);
      h.push(idx[idx.length - 1]);
    } else {
      logits = native.prefill(this.model.handle, Int32Array.from(idx), this.params.vocab_size);
      this._history = Array.from(idx);
    }
    this.lastGpuMs = native.modelLastGpuMs(this.model.handle);
    return logits;
  }

  // Greedy continuation entirely on the device: ids of `steps` tokens after `token`.
  decodeGreedy(token, steps) {
    const ids = native.decodeGreedy(this.model.handle, token, steps);
    this._history = this._history.concat([token], Array.from(ids.slice(0, steps - 1)));
    this.lastGpuMs = native.modelLastGpuMs(this.model.handle);
    return ids;
  }

  // Sampled continuation on the device: one token per entry of `draws` (uniform numbers in
  // [0, 1), what the reference takes from Math.random()), chosen as generate() chooses
  // (model.js:81-85) without reading the logits back.
  decodeSample(token, topK, temperature, draws) {
    const u = Float64Array.from(draws);
    const ids = native.decodeSample(this.model.handle, token, topK, temperature, u);
    this._history = this._history.concat([token], Array.from(ids.slice(0, u.length - 1)));
    this.lastGpuMs = native.modelLastGpuMs(this.model.handle);
    return ids;
  }

  // The reference's pass list (model.js:118-240) built block by block from separately
  // uploaded weights and replayed through the per-block entry points.
  // `vocab` (optional) passes the table as the reference holds it: { vocab_chunk_size, embdBuffers, deEmbeddingsBuffers }.
  async runBlocks(idx, weights, vocab) {
    const { n_embd, n_head, head_size, n_layer, vocab_size, hidden_size, attention_scale } = this.params;
    const seq_length = idx.length;
    const passesAll = [];
    let intermediateBuffer, residualBuffer;
    const push = ({ passes, resultBuffer }) => {
      passesAll.push(...passes);
      return resultBuffer;
    };
    const chunkSize = vocab ? vocab.vocab_chunk_size : vocab_size;
    const embdBuffers = vocab ? vocab.embdBuffers : [weights.wte], deEmbeddingsBuffers = vocab ? vocab.deEmbeddingsBuffers : [weights.wte];
    intermediateBuffer = residualBuffer = push(G.EmbedBlock.newInstance(idx, seq_length, n_embd, chunkSize, embdBuffers, weights.wpe, G.ResidualBlock));
    for (let i = 0; i < n_layer; i++) {
      const b = weights.layers[i];
      intermediateBuffer = push(G.LayerNormBlock.newInstance(seq_length, n_embd, intermediateBuffer, b.normAttentionGammaBuffer, b.normAttentionBetaBuffer));
      intermediateBuffer = push(G.AttentionBlock.newFusedInstance(seq_length, n_embd, attention_scale, n_head, head_size, intermediateBuffer,
        b.qkvWeightArray[0], b.qkvBiasArray[0], b.qkvWeightArray[1], b.qkvBiasArray[1], b.qkvWeightArray[2], b.qkvBiasArray[2],
        b.linearWeightsBuffer, b.linearBiasBuffer, G.FastMatMulBlock, G.SoftmaxBlock));
      intermediateBuffer = residualBuffer = push(G.ResidualBlock.newInstance(seq_length, n_embd, intermediateBuffer, residualBuffer));
      intermediateBuffer = push(G.LayerNormBlock.newInstance(seq_length, n_embd, intermediateBuffer, b.normLinearGammaBuffer, b.normLinearBetaBuffer));
      intermediateBuffer = push(G.FastMatMulBlock.newInstance(seq_length, hidden_size, n_embd, intermediateBuffer, b.firstLayerWeightsBuffer, b.firstLayerBiasBuffer));
      intermediateBuffer = push(G.GeluBlock.newInstance(seq_length, hidden_size, intermediateBuffer));
      intermediateBuffer = push(G.FastMatMulBlock.newInstance(seq_length, n_embd, hidden_size, intermediateBuffer, b.secondLayerWeightsBuffer, b.secondLayerBiasBuffer));
      intermediateBuffer = residualBuffer = push(G.ResidualBlock.newInstance(seq_length, n_embd, intermediateBuffer, residualBuffer));
    }
    if (this.externalBuffer) {
      passesAll.push({ flag: "copy", src: intermediateBuffer, srcOffset: 0, dst: this.externalBuffer, dstOffset: 0, size: this.bufferSize(seq_length, n_embd) });
    }
    intermediateBuffer = push(G.LayerNormBlock.newInstance(seq_length, n_embd, intermediateBuffer, weights.normGammaBuffer, weights.normBetaBuffer));
    const resultBuffer = push(G.DeEmbedBlock.newInstance(n_embd, vocab_size, chunkSize * deEmbeddingsBuffers.length, seq_length, chunkSize, intermediateBuffer, deEmbeddingsBuffers));
    runPasses(passesAll);
    const out = resultBuffer.download();
    G.clearOperationCache();
    return out;
  }

  // Uploads a {name: Float32Array} weight directory as separate buffers with the
  // reference's load-time transforms (model.js:339-482), for runBlocks.
  loadBlockWeights(tensors) {
    const { n_embd: d, n_layer, n_ctx, vocab_size, hidden_size } = this.params;
    const get = (n) => tensors[n];
    const T = (data, dims) => this.initTensor(data, dims, ["storage"]);
    const layers = [];
    for (let i = 0; i < n_layer; i++) {
      const p = `transformer.h.${i}.`;
      // fetchAndSplitQKVWeightTensors: columns 0..d, d..2d, 2d..3d of c_attn [d, 3d]
      const w = get(p + "attn.c_attn.weight"), b = get(p + "attn.c_attn.bias");
      const split = [0, 1, 2].map((part) => {
        const out = new Float32Array(d * d);
        for (let k = 0; k < d; k++) out.set(w.subarray(k * 3 * d + part * d, k * 3 * d + (part + 1) * d), k * d);
        return T(out, [d, d]);
      });
      layers.push({
        normAttentionGammaBuffer: T(get(p + "ln_1.weight"), [d]), normAttentionBetaBuffer: T(get(p + "ln_1.bias"), [d]),
        qkvWeightArray: split, qkvBiasArray: [0, 1, 2].map((part) => T(b.subarray(part * d, (part + 1) * d), [d])),
        linearWeightsBuffer: T(get(p + "attn.c_proj.weight"), [d, d]), linearBiasBuffer: T(get(p + "attn.c_proj.bias"), [d]),
        normLinearGammaBuffer: T(get(p + "ln_2.weight"), [d]), normLinearBetaBuffer: T(get(p + "ln_2.bias"), [d]),
        firstLayerWeightsBuffer: T(get(p + "mlp.c_fc.weight"), [d, hidden_size]), firstLayerBiasBuffer: T(get(p + "mlp.c_fc.bias"), [hidden_size]),
        secondLayerWeightsBuffer: T(get(p + "mlp.c_proj.weight"), [hidden_size, d]), secondLayerBiasBuffer: T(get(p + "mlp.c_proj.bias"), [d]),
      });
    }
    return {
      layers, wte: T(get("transformer.wte.weight"), [vocab_size, d]), wpe: T(get("transformer.wpe.weight"), [n_ctx, d]),
      normGammaBuffer: T(get("transformer.ln_f.weight"), [d]), normBetaBuffer: T(get("transformer.ln_f.bias"), [d]),
    };
  }

  // loadModel and the loaders it calls keep the reference's names, order and return shapes
  // (model.js:270-488). A "buffer" they return is a descriptor { name, dims } of a tensor that
  // now lives in the library's model (wgpt_model_set_tensor copies the data in); the Q/K/V
  // entries are column ranges of the fused c_attn, which the library keeps whole.
  async loadModel(folder) {
    if (this.initialized) return console.error("Model already loaded");
    const weightsFolder = folder;
    const params = await this.loadParameters(weightsFolder);
    const names = this._tensors ? Object.keys(this._tensors) : undefined;
    const packed = !!names && names.some((n) => n.endsWith(".weight.q"));
    this._quantise = !packed && (this._quantize || params.quantize) === "int8";
    const handle = native.modelCreate(params.n_layer, params.n_head, params.n_embd, params.n_ctx, params.vocab_size, packed || this._quantise ? 1 : 0, params.max_prefill || 0, this._flags);
    this._loading = { handle, params, packed };
    let output;
    try {
      const { embeddingsBuffers, deEmbeddingsBuffers } = await this.loadEmbeddings(params, weightsFolder);
      const { posEmbdBuffer } = await this.loadPositionalEmbeddings(params, weightsFolder);
      const layer_buffers = await this.loadLayers(params, weightsFolder);
      const { normGammaBuffer, normBetaBuffer } = await this.loadFinalLayerNorm(params, weightsFolder);
      native.modelFinalize(handle);
      output = { handle, layer_buffers, embeddingsBuffers, deEmbeddingsBuffers, posEmbdBuffer, normGammaBuffer, normBetaBuffer };
    } catch (e) {
      native.modelDestroy(handle);
      throw e;
    } finally {
      this._loading = undefined;
    }
    return [output, params];
  }

  async loadParameters(weightsFolder) {
    const params = this._paramsIn ? Object.assign({}, this._paramsIn) : JSON.parse(fs.readFileSync(path.join(weightsFolder, "params_gpt.json"), "utf8"));
    // model.js:294-297
    if (params.n_embd % 4 !== 0) throw new Error("Model load failed: n_embd must be divisible by 4.");
    if (params.n_embd % params.n_head !== 0) throw new Error("Model load failed: n_embd must be divisible by n_head.");
    if ((params.n_embd / params.n_head) % 4 !== 0) throw new Error("Model load failed: n_embd / n_head must be divisible by 4.");
    // the vocabulary is never split here: one buffer, one launch
    params.vocab_chunk_size = params.vocab_size;
    params.vocab_chunk_instances = 1;
    params.head_size = params.n_embd / params.n_head;
    params.hidden_size = params.n_embd * 4;
    params.attention_scale = 1 / Math.sqrt(params.n_embd / params.n_head);
    params.bias = params.bias == undefined ? true : params.bias;
    // model.js:325-332: the soft limits, against this device's largest buffer (all of HBM)
    const maxBufferSize = (this.device ? this.device.limits.maxStorageBufferBindingSize : Infinity) / 4;
    if (params.n_embd * params.n_ctx > maxBufferSize) console.warn("Model load failed: n_embd * n_ctx must be less than maxStorageBufferBindingSize.");
    if (params.n_embd * params.hidden_size > maxBufferSize) console.warn("Model load failed: n_embd * hidden_size must be less than maxStorageBufferBindingSize.");
    if (params.n_ctx * params.n_ctx * params.n_head > maxBufferSize) console.warn("Model load failed: n_ctx * n_ctx must be less than maxStorageBufferBindingSize.");
    if (params.n_embd * params.n_embd * 3 > maxBufferSize) console.warn("Model load failed: n_embd * n_embd * 3 must be less than maxStorageBufferBindingSize.");
    return params;
  }

  // model.js:339-367. One table serves the gather and the vocabulary projection (row-major wte has
  // the contraction index contiguous), so both lists hold the same single descriptor.
  async loadEmbeddings(params, weightsFolder) {
    const wte = await this.fetchAndInitTensor(`${weightsFolder}/transformer.wte.weight_gpt.bin`, [params.vocab_size, params.n_embd], ["copy_from"]);
    return { embeddingsBuffers: [wte], deEmbeddingsBuffers: [wte] };
  }

  async loadPositionalEmbeddings(params, weightsFolder) {
    const posEmbdBuffer = await this.fetchAndInitTensor(`${weightsFolder}/transformer.wpe.weight_gpt.bin`, [params.n_ctx, params.n_embd], ["copy_from"]);
    return { posEmbdBuffer };
  }

  async loadFinalLayerNorm(params, weightsFolder) {
    const prefix = `${weightsFolder}/transformer.ln_f.`;
    const [normGammaBuffer, normBetaBuffer] = await Promise.all([
      this.fetchAndInitTensor(`${prefix}weight_gpt.bin`, [params.n_embd], ["storage"]),
      this.fetchAndInitTensor(`${prefix}bias_gpt.bin`, [params.n_embd], ["storage"]),
    ]);
    return { normGammaBuffer, normBetaBuffer };
  }

  async loadLayers(params, weightsFolder) {
    const layerPromises = [];
    for (let i = 0; i < params.n_layer; i++) layerPromises.push(this.loadLayer(params, weightsFolder, i));
    return await Promise.all(layerPromises);
  }

  async loadLayer(params, weightsFolder, layerIndex) {
    const prefix = `${weightsFolder}/transformer.h.${layerIndex}.`;
    const d = params.n_embd, hid = params.hidden_size;
    const [normAttentionGammaBuffer, normAttentionBetaBuffer, qkvWeightArray, qkvBiasArray, linearWeightsBuffer, linearBiasBuffer,
      normLinearGammaBuffer, normLinearBetaBuffer, firstLayerWeightsBuffer, firstLayerBiasBuffer, secondLayerWeightsBuffer, secondLayerBiasBuffer] = await Promise.all([
      this.fetchAndInitTensor(`${prefix}ln_1.weight_gpt.bin`, [d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}ln_1.bias_gpt.bin`, [d], ["storage"]),
      this.fetchAndSplitQKVWeightTensors(`${prefix}attn.c_attn.weight_gpt.bin`, [d, 3 * d], ["storage"]),
      this.fetchAndSplitQKVBiasTensors(`${prefix}attn.c_attn.bias_gpt.bin`, [d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}attn.c_proj.weight_gpt.bin`, [d, d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}attn.c_proj.bias_gpt.bin`, [d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}ln_2.weight_gpt.bin`, [d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}ln_2.bias_gpt.bin`, [d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}mlp.c_fc.weight_gpt.bin`, [d, hid], ["storage"]),
      this.fetchAndInitTensor(`${prefix}mlp.c_fc.bias_gpt.bin`, [hid], ["storage"]),
      this.fetchAndInitTensor(`${prefix}mlp.c_proj.weight_gpt.bin`, [hid, d], ["storage"]),
      this.fetchAndInitTensor(`${prefix}mlp.c_proj.bias_gpt.bin`, [d], ["storage"]),
    ]);
    return { normAttentionGammaBuffer, normAttentionBetaBuffer, qkvWeightArray, qkvBiasArray, linearWeightsBuffer, linearBiasBuffer,
      normLinearGammaBuffer, normLinearBetaBuffer, firstLayerWeightsBuffer, firstLayerBiasBuffer, secondLayerWeightsBuffer, secondLayerBiasBuffer };
  }

  // model.js:456-482: the reference cuts c_attn [d, 3d] into three [d, d] matrices (and its bias into
  // three vectors) on the host. Here the fused tensor goes to the library as it is and Q, K, V are
  // its column ranges 0..d, d..2d, 2d..3d, which is what the three descriptors say.
  async fetchAndSplitQKVWeightTensors(url, dims, ops) {
    const fused = await this.fetchAndInitTensor(url, [dims[0], 3 * dims[0]], ops);
    return [0, 1, 2].map((part) => ({ name: fused.name, dims: [dims[0], dims[0]], columns: [part * dims[0], (part + 1) * dims[0]] }));
  }

  async fetchAndSplitQKVBiasTensors(url, dims, ops) {
    const fused = await this.fetchAndInitTensor(url, [3 * dims[0]], ops);
    return [0, 1, 2].map((part) => ({ name: fused.name, dims: [dims[0]], columns: [part * dims[0], (part + 1) * dims[0]] }));
  }

  // model.js:484-488: reads <name>_gpt.bin (or the in-memory tensor of that name) and hands it to the
  // model being loaded. A linear weight goes in as it is, as its packed int8 words and column scales
  // when the directory holds those, or quantised here when the model was opened with quantize: "int8".
  async fetchAndInitTensor(url, dims, ops) {
    const { handle, params, packed } = this._loading;
    const name = path.basename(url).replace(/_gpt\.bin$/, "");
    const linear = /^transformer\.h\.\d+\.(attn\.c_attn|attn\.c_proj|mlp\.c_fc|mlp\.c_proj)\.weight$/.test(name);
    const fetch = (n) => (this._tensors ? this._tensors[n] : this.readTensor(path.dirname(url), n, params));
    if (linear && packed) {
      native.modelSetTensor(handle, name + ".q", fetch(name + ".q"));
      native.modelSetTensor(handle, name + ".scale", fetch(name + ".scale"));
    } else if (linear && this._quantise) {
      const { quantizedMatrix, scale } = quantizeMatrix(fetch(name), dims[0], dims[1]);
      native.modelSetTensor(handle, name + ".q", quantizedMatrix);
      native.modelSetTensor(handle, name + ".scale", scale);
    } else {
      native.modelSetTensor(handle, name, fetch(name));
    }
    return { name, dims };
  }

  directoryNames(params) {
    const names = ["transformer.wte.weight", "transformer.wpe.weight"];
    for (let i = 0; i < params.n_layer; i++) {
      for (const s of ["ln_1.weight", "ln_1.bias", "attn.c_attn.weight", "attn.c_attn.bias", "attn.c_proj.weight", "attn.c_proj.bias",
        "ln_2.weight", "ln_2.bias", "mlp.c_fc.weight", "mlp.c_fc.bias", "mlp.c_proj.weight", "mlp.c_proj.bias"]) names.push(`transformer.h.${i}.${s}`);
    }
    return names.concat(["transformer.ln_f.weight", "transformer.ln_f.bias"]);
  }

  // Shape of a tensor file as the forward path wants it: linear weights [in, out], the layout
  // other/conversion_scripts/*.py write for HF GPT-2 Conv1D modules (model.js:404-417).
  tensorShape(name, params) {
    const d = params.n_embd;
    const linear = { "attn.c_attn.weight": [1, 3], "attn.c_proj.weight": [1, 1], "mlp.c_fc.weight": [1, 4], "mlp.c_proj.weight": [4, 1] };
    if (name === "transformer.wte.weight") return [params.vocab_size, d];
    if (name === "transformer.wpe.weight") return [params.n_ctx, d];
    const rest = name.startsWith("transformer.h.") ? name.split(".").slice(3).join(".") : name;
    if (linear[rest]) return [linear[rest][0] * d, linear[rest][1] * d];
    const w = rest.replace(/\.bias$/, ".weight");
    if (rest.endsWith(".bias") && linear[w]) return [linear[w][1] * d];
    return [d];
  }

  // One <name>_gpt.bin. Two variations of the directory that earlier versions of the reference
  // handled (condensed/condensed.js:1755-1783) are accepted through params_gpt.json:
  // "bias": false - bias files are absent and read as zeros; "linear_layout": "out_in" - the four
  // linear weights are stored [out, in] (torch nn.Linear, nanoGPT) and are transposed here.
  readTensor(folder, name, params) {
    const shape = this.tensorShape(name, params);
    const count = shape.reduce((a, b) => a * b, 1);
    if (name.endsWith(".bias") && params.bias === false) return G.zeros(count);
    const data = this.fetchBin(path.join(folder, `${name}_gpt.bin`));
    if (data.length !== count) throw new Error(`Model load failed: ${name}_gpt.bin holds ${data.length} values, expected ${count}.`);
    if (shape.length === 2 && params.linear_layout === "out_in" && !name.startsWith("transformer.w")) return G.transpose(data, shape[1], shape[0]);
    return data;
  }

  fetchBin(file) {
    const b = fs.readFileSync(file);
    return new Float32Array(b.buffer, b.byteOffset, b.byteLength / 4);
  }

  initTensor(data, dims, ops) {
    const buffer = initTensor(data, dims);
    this.unloadDeletionStack.push(buffer);
    return buffer;
  }

  unloadBuffers() {
    this.unloadDeletionStack.map((buffer) => buffer.destroy());
    this.unloadDeletionStack = [];
    if (this.model) native.modelDestroy(this.model.handle);
    this.model = undefined;
    this.initialized = false;
  }

  bufferSize(dimX, dimY = 1, dimZ = 1) {
    return Math.ceil((dimX * dimY * dimZ * Float32Array.BYTES_PER_ELEMENT) / this.minBufferOffset) * this.minBufferOffset;
  }
}

module.exports = { GPT };
