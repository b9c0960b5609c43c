// Block singletons, lifecycle helpers and the host-side helper functions of the
// reference's globals.js, for Node (CommonJS) instead of <script> globals.
"use strict";
const blocks = require("./instructions.js");

const FastMatMulBlock = new blocks.FastMatMulBlockClass();
const AttentionBlock = new blocks.AttentionBlockClass();
const ResidualBlock = new blocks.ResidualBlockClass();
const EmbedBlock = new blocks.EmbedBlockClass();
const DeEmbedBlock = new blocks.DeEmbedBlockClass();
const GeluBlock = new blocks.GeluBlockClass();
const LayerNormBlock = new blocks.LayerNormBlockClass();
const SoftmaxBlock = new blocks.SoftmaxBlockClass();

// Needed for deletion (globals.js:11).
const operations = [FastMatMulBlock, AttentionBlock, ResidualBlock, EmbedBlock, DeEmbedBlock, GeluBlock, LayerNormBlock, SoftmaxBlock];

function initializeOperations(device) {
  for (const operation of operations) operation.initialize(device);
}
function destroyOperationBuffers() {
  for (const operation of operations) operation.destroyBuffers();
}
function clearOperationCache() {
  for (const operation of operations) operation.clearBufferCache();
}
function destroyOperations() {
  for (const operation of operations) operation.destroy();
}

// Usage-flag names accepted by initTensor / initBuffer (globals.js:29-35). Every
// buffer is plain device memory here, so the flags carry no meaning beyond being accepted.
const bufferUsageDict = { copy_from: 1, copy_to: 2, storage: 4, uniform: 8, map_read: 16 };

// ---------------- Helper functions ----------------

const wgSize = (dim, size) => Math.ceil(dim / size);

// Inverse-CDF sampling (globals.js:47-57).
function sampleFromDistribution(probs, rand = Math.random()) {
  let cumulative = 0;
  for (let i = 0; i < probs.length; i++) {
    cumulative += probs[i];
    if (rand < cumulative) return i;
  }
  return probs.length - 1;
}

// float64 softmax with the temperature inside the exponent (globals.js:59-64).
function cpuSoftmax(logits, temperature = 1.0) {
  let maxLogit = -Infinity;
  for (const l of logits) if (l > maxLogit) maxLogit = l;
  const e = Array.from(logits, (l) => Math.exp((l - maxLogit) / temperature));
  let sum = 0;
  for (const v of e) sum += v;
  return e.map((v) => v / sum);
}

// top_k largest by a stable descending sort: ties keep the lower index first
// (globals.js:66-74). top_k = 1 is a single linear scan.
function selectTopK(probs, top_k) {
  let topKIndices;
  if (top_k === 1) {
    let best = 0;
    for (let i = 1; i < probs.length; i++) if (probs[i] > probs[best]) best = i;
    topKIndices = [best];
  } else {
    topKIndices = Array.from(probs, (value, index) => ({ value, index }))
      .sort((a, b) => b.value - a.value || a.index - b.index)
      .slice(0, top_k)
      .map((p) => p.index);
  }
  return { topKIndices, topKProbs: topKIndices.map((i) => probs[i]) };
}

// ----------------------- Matrix operations -----------------------

const zeros = (dim) => new Float32Array(dim);

function transpose(array, input_rows, input_cols) {
  if (array.length !== input_rows * input_cols) throw new Error("Transpose dims failed");
  const out = new Float32Array(array.length);
  for (let row = 0; row < input_rows; row++) {
    for (let col = 0; col < input_cols; col++) out[col * input_rows + row] = array[row * input_cols + col];
  }
  return out;
}

function formatAsMatrix(floatArray, dimA, dimB) {
  const rows = [];
  for (let i = 0; i < dimA; i++) rows.push(floatArray.slice(i * dimB, (i + 1) * dimB));
  return rows;
}

module.exports = {
  FastMatMulBlock, AttentionBlock, ResidualBlock, EmbedBlock, DeEmbedBlock, GeluBlock, LayerNormBlock, SoftmaxBlock,
  operations, initializeOperations, destroyOperationBuffers, clearOperationCache, destroyOperations, bufferUsageDict,
  wgSize, sampleFromDistribution, cpuSoftmax, selectTopK, zeros, transpose, formatAsMatrix,
};
