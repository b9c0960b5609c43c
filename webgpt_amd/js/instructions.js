// Instruction blocks: the operator API of the reference's instructions.js over the
// HIP library. Each newInstance(...) takes the reference's arguments in the
// reference's order and returns { resultBuffer, passes }; a pass is
// { flag: "compute", op, args } or { flag: "copy", src, srcOffset, dst, dstOffset, size }
// and is executed by runPasses (the command-encoding loop of model.js:245-257),
// which calls the C ABI instead of a WebGPU command encoder.
"use strict";
const native = require("./native.js");

// A device buffer handle (what the reference holds as a GPUBuffer).
class DeviceBuffer {
  constructor(dims) {
    this.dims = dims.slice();
    this.size = 4 * dims.reduce((a, b) => a * b, 1);
    this.handle = native.alloc(this.size);
    this.destroyed = false;
  }
  destroy() {
    if (!this.destroyed) native.free(this.handle);
    this.destroyed = true;
    if (this.rows) {  // row form of a transposed vocabulary chunk (DeEmbedBlock)
      this.rows.destroy();
      this.rows = null;
    }
  }
  upload(typedArray, offset = 0) {
    native.upload(this.handle, offset, typedArray);
  }
  download(offset = 0, size = this.size) {
    return new Float32Array(native.download(this.handle, offset, size));
  }
}

// Stands in for the GPUDevice the reference threads through its blocks.
class Device {
  constructor(index = 0) {
    native.init(index);  // throws when no gfx950 device exists: there is no fallback
    const info = native.deviceInfo();
    this.name = info.name;
    this.computeUnits = info.computeUnits;
    // no binding-size limit exists here: all of HBM is addressable from a kernel
    this.limits = { maxStorageBufferBindingSize: info.hbmBytes, maxBufferSize: info.hbmBytes };
  }
  sync() {
    native.sync();
  }
  destroy() {
    native.shutdown();
  }
}

function initTensor(data, dims) {
  const buf = new DeviceBuffer(dims);
  buf.upload(data);
  return buf;
}

const compute = (op, ...args) => ({ flag: "compute", op, args });

// Base class (instructions.js:7-139). Pipelines and bind groups have no counterpart;
// the double-buffered result-buffer pool is kept: buffers made during one run are
// released by the clearBufferCache() after the next run.
class Block {
  constructor() {
    this.name = "";
  }
  initialize(device) {
    this.device = device;
    this.boundBufferCache = [];
    this.unboundBufferCache = [];
  }
  initResultBuffer(dims) {
    return this.initBuffer(["storage", "copy_from"], dims);
  }
  initBuffer(ops, dims) {
    this.bufferSize(dims[0], dims[1] || 1);
    const buffer = new DeviceBuffer(dims);
    this.boundBufferCache.push(buffer);
    return buffer;
  }
  bufferSize(dimA, dimB = 1) {
    const size = dimA * dimB * Float32Array.BYTES_PER_ELEMENT;
    if (size > this.device.limits.maxStorageBufferBindingSize) throw new Error("Buffer size exceeds GPU limit.");
    return size;
  }
  clearBufferCache() {
    this.unboundBufferCache.forEach((b) => b.destroy());
    this.unboundBufferCache = this.boundBufferCache;
    this.boundBufferCache = [];
  }
  destroyBuffers() {
    this.unboundBufferCache.concat(this.boundBufferCache).forEach((b) => b.destroy());
    this.unboundBufferCache = [];
    this.boundBufferCache = [];
  }
  destroy() {
    this.destroyBuffers();
  }
}

class FastMatMulBlockClass extends Block {
  constructor() {
    super();
    this.name = "fastMatMul";
  }
  newInstance(rows, cols, shared, inputBuffer, weightsBuffer, biasBuffer) {
    if (cols % 8 !== 0) throw new Error("Cols must be divisible by 16.");
    const resultBuffer = this.initResultBuffer([rows, cols]);
    return {
      resultBuffer,
      passes: [compute("wgpt_matmul_bias", rows, cols, shared, inputBuffer.handle, weightsBuffer.handle, biasBuffer ? biasBuffer.handle : 0, resultBuffer.handle)],
    };
  }
  // other/int8-gemm.js as a block: packed int8 words + per-column scales.
  newInt8Instance(rows, cols, shared, inputBuffer, packedWeightsBuffer, scaleBuffer, biasBuffer) {
    if (cols % 8 !== 0) throw new Error("Cols must be divisible by 16.");
    const resultBuffer = this.initResultBuffer([rows, cols]);
    return {
      resultBuffer,
      passes: [compute("wgpt_matmul_bias_i8", rows, cols, shared, inputBuffer.handle, packedWeightsBuffer.handle, scaleBuffer.handle, biasBuffer ? biasBuffer.handle : 0, resultBuffer.handle)],
    };
  }
}

class ResidualBlockClass extends Block {
  constructor() {
    super();
    this.name = "residual";
  }
  newInstance(rows, cols, outputBuf, residualBuf) {
    if (cols % 4 !== 0) throw new Error("Cols must be divisible by 4.");
    const resultBuffer = this.initResultBuffer([rows, cols]);
    return { resultBuffer, passes: [compute("wgpt_residual", rows, cols, outputBuf.handle, residualBuf.handle, resultBuffer.handle)] };
  }
}

class LayerNormBlockClass extends Block {
  constructor() {
    super();
    this.name = "layerNorm";
  }
  newInstance(rows, cols, inputBuffer, gammaBuffer, betaBuffer) {
    if (cols % 4 !== 0) throw new Error("Cols must be divisible by 4.");
    const resultBuffer = this.initResultBuffer([rows, cols]);
    return { resultBuffer, passes: [compute("wgpt_layernorm", rows, cols, inputBuffer.handle, gammaBuffer.handle, betaBuffer.handle, resultBuffer.handle)] };
  }
}

class SoftmaxBlockClass extends Block {
  constructor() {
    super();
    this.name = "softmax";
  }
  // transpose: the same values stored as [cols, rows] (instructions.js:594)
  newInstance(rows, cols, inputBuffer, transpose = false) {
    const resultBuffer = this.initResultBuffer(transpose ? [cols, rows] : [rows, cols]);
    return { resultBuffer, passes: [compute(transpose ? "wgpt_softmax_t" : "wgpt_softmax", rows, cols, inputBuffer.handle, resultBuffer.handle)] };
  }
}

class GeluBlockClass extends Block {
  constructor() {
    super();
    this.name = "gelu";
  }
  newInstance(rows, cols, inputBuf) {
    if (cols % 4 !== 0) throw new Error("Cols must be divisible by 4.");
    const resultBuffer = this.initResultBuffer([rows, cols]);
    return { resultBuffer, passes: [compute("wgpt_gelu", rows, cols, inputBuf.handle, resultBuffer.handle)] };
  }
}

class EmbedBlockClass extends Block {
  constructor() {
    super();
    this.name = "embed";
  }
  // embdBuffers is either the single un-chunked [V, d] table (one fused gather + add) or the reference's list of
  // zero-padded [vocab_chunk_size, d] chunks (model.js:348-361): then token i is row idx[i] % vocab_chunk_size of chunk
  // floor(idx[i] / vocab_chunk_size), copied row by row, and the positional rows are added by the ResidualBlock, as
  // the reference does (instructions.js:795-821).
  newInstance(idx, seq_length, n_embd, vocab_chunk_size, embdBuffers, posEmbdBuffer, ResidualBlock) {
    if (embdBuffers.length === 1) {
      const ids = Int32Array.from(idx);
      const resultBuffer = this.initResultBuffer([seq_length, n_embd]);
      return {
        resultBuffer,
        passes: [compute("wgpt_embed", ids, seq_length, n_embd, embdBuffers[0].dims[0], embdBuffers[0].handle, posEmbdBuffer.handle, resultBuffer.handle)],
      };
    }
    const row = 4 * n_embd;
    const embdOutputBuffer = this.initBuffer(["storage", "copy_to"], [seq_length, n_embd]);
    const posEmbdOutputBuffer = this.initBuffer(["storage", "copy_to"], [seq_length, n_embd]);
    const passes = [];
    for (let i = 0; i < seq_length; i++) {
      const chunk = Math.floor(idx[i] / vocab_chunk_size);
      if (!(idx[i] >= 0) || chunk >= embdBuffers.length) throw new Error("token id outside the embedding chunks");
      passes.push({ flag: "copy", src: embdBuffers[chunk], srcOffset: row * (idx[i] % vocab_chunk_size), dst: embdOutputBuffer, dstOffset: row * i, size: row });
    }
    passes.push({ flag: "copy", src: posEmbdBuffer, srcOffset: 0, dst: posEmbdOutputBuffer, dstOffset: 0, size: row * seq_length });
    const res = ResidualBlock.newInstance(seq_length, n_embd, embdOutputBuffer, posEmbdOutputBuffer);
    return { resultBuffer: res.resultBuffer, passes: passes.concat(res.passes) };
  }
}

class DeEmbedBlockClass extends Block {
  constructor() {
    super();
    this.name = "deembed";
  }
  // deEmbeddingsBuffers is either the single [V, d] table (no host transposes, no chunk copies) or the reference's
  // list of transposed, zero-padded [d, vocab_chunk_size] chunks (model.js:362-363). A chunk is turned back into rows
  // on the device the first time it is seen (wgpt_transpose; the row form is kept with the buffer, which the
  // reference also makes once, at load), and every chunk's logits go to their offset in the result, the last copy
  // dropping the padding columns (instructions.js:873-880). Same kernel row by row: same logits bit for bit.
  newInstance(n_embd, vocab_size, padded_vocab_size, seq_length, vocab_chunk_size, embedBuffer, deEmbeddingsBuffers) {
    const resultBuffer = this.initBuffer(["map_read", "copy_to"], [vocab_size]);
    if (deEmbeddingsBuffers.length === 1 && deEmbeddingsBuffers[0].dims[0] === vocab_size) {
      return { resultBuffer, passes: [compute("wgpt_deembed", n_embd, vocab_size, seq_length, embedBuffer.handle, deEmbeddingsBuffers[0].handle, resultBuffer.handle)] };
    }
    const passes = [];
    for (let i = 0; i < deEmbeddingsBuffers.length; i++) {
      const chunkBuffer = deEmbeddingsBuffers[i];
      if (chunkBuffer.dims[0] !== n_embd || chunkBuffer.dims[1] !== vocab_chunk_size) throw new Error("a de-embedding chunk must be [n_embd, vocab_chunk_size]");
      if (!chunkBuffer.rows) {
        chunkBuffer.rows = new DeviceBuffer([vocab_chunk_size, n_embd]);
        native.wgpt_transpose(n_embd, vocab_chunk_size, chunkBuffer.handle, chunkBuffer.rows.handle);
      }
      const valid = Math.min(vocab_chunk_size, vocab_size - i * vocab_chunk_size);
      if (valid <= 0) break;
      const chunkResultBuffer = this.initResultBuffer([valid]);
      passes.push(compute("wgpt_deembed", n_embd, valid, seq_length, embedBuffer.handle, chunkBuffer.rows.handle, chunkResultBuffer.handle));
      passes.push({ flag: "copy", src: chunkResultBuffer, srcOffset: 0, dst: resultBuffer, dstOffset: 4 * i * vocab_chunk_size, size: 4 * valid });
    }
    return { resultBuffer, passes };
  }
}

class AttentionBlockClass extends Block {
  constructor() {
    super();
    this.name = "attention";
  }
  newFusedInstance(seq_length, n_embd, attentionDotProductScale, n_head, head_size, inputBuffer, qWeightsBuffer, qBiasBuffer, kWeightsBuffer, kBiasBuffer, vWeightsBuffer, vBiasBuffer, linearWeightsBuffer, linearBiasBuffer, FastMatMulBlock, SoftmaxBlock) {
    const resultBuffer = this.initResultBuffer([seq_length, n_embd]);
    const handles = [inputBuffer, qWeightsBuffer, qBiasBuffer, kWeightsBuffer, kBiasBuffer, vWeightsBuffer, vBiasBuffer, linearWeightsBuffer, linearBiasBuffer].map((b) => b.handle);
    return { resultBuffer, passes: [compute("wgpt_attention", seq_length, n_embd, attentionDotProductScale, n_head, head_size, ...handles, resultBuffer.handle)] };
  }
}

// The command-encoding loop of model.js:245-257 over the HIP library.
function runPasses(passes) {
  for (const pass of passes) {
    if (pass.flag === "compute") {
      native[pass.op](...pass.args);
    } else if (pass.flag === "copy") {
      native.copy(pass.dst.handle, pass.dstOffset, pass.src.handle, pass.srcOffset, pass.size);
    } else {
      throw new Error(`unknown pass flag ${pass.flag}`);
    }
  }
}

module.exports = {
  DeviceBuffer, Device, initTensor, Block, runPasses,
  FastMatMulBlockClass, ResidualBlockClass, LayerNormBlockClass, SoftmaxBlockClass, GeluBlockClass, EmbedBlockClass, DeEmbedBlockClass, AttentionBlockClass,
};
