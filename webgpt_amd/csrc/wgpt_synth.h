// Deterministic synthetic tensors for the GPT-2 forward path.
//
// Everything is integer arithmetic (32-bit wrap-around hashing, 24-bit uniforms
// summed exactly) until one final double multiply and one rounding to float, so
// the C, numpy and JavaScript (Math.imul) implementations produce bit-identical
// weights, token ids, int8 values and scales from (seed, tensor_id, index).
//
// The weight files this stands in for are the reference's per-tensor
// little-endian f32 dumps (other/conversion_scripts/convert_pretrained_pytorch.py:18-22).
#ifndef WGPT_SYNTH_H
#define WGPT_SYNTH_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

// 32-bit finalizer ("lowbias32"): bijective, good avalanche, only xor-shift and
// wrap-around multiplies, which JavaScript reproduces with Math.imul and >>> 0.
static inline uint32_t wgpt_mix32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7feb352dU;
  x ^= x >> 15;
  x *= 0x846ca68bU;
  x ^= x >> 16;
  return x;
}

// Key of one tensor: depends on the run seed and the tensor id only.
static inline uint32_t wgpt_tensor_key(uint32_t seed, uint32_t tensor_id) {
  return wgpt_mix32(seed * 0x9e3779b1U + tensor_id * 0x85ebca77U + 0x165667b1U);
}

// Key of one element of a tensor.
static inline uint32_t wgpt_elem_key(uint32_t tkey, uint32_t index) {
  return wgpt_mix32(tkey ^ wgpt_mix32(index + 0x27d4eb2fU));
}

// j-th 32-bit draw of an element.
static inline uint32_t wgpt_draw(uint32_t ekey, uint32_t j) {
  return wgpt_mix32(ekey + j * 0x9e3779b9U);
}

// Approximately N(0, std): Irwin-Hall sum of twelve 24-bit uniforms (variance 1
// after centring), computed exactly in integers, then one double multiply.
static inline float wgpt_synth_normal_at(uint32_t tkey, uint32_t index, double std_) {
  uint32_t e = wgpt_elem_key(tkey, index);
  int32_t sum = 0;
  for (uint32_t j = 0; j < 12; ++j) sum += (int32_t)(wgpt_draw(e, j) >> 8);
  sum -= 6 * (1 << 24);
  return (float)((double)sum * (std_ / 16777216.0));
}

// Uniform token id in [0, vocab).
static inline int32_t wgpt_synth_token_at(uint32_t tkey, uint32_t index, uint32_t vocab) {
  return (int32_t)(wgpt_draw(wgpt_elem_key(tkey, index), 0) % vocab);
}

// Uniform signed byte in [-127, 127].
static inline int32_t wgpt_synth_int8_at(uint32_t tkey, uint32_t index) {
  return (int32_t)(wgpt_draw(wgpt_elem_key(tkey, index), 0) % 255U) - 127;
}

// Uniform float in [lo, hi): 24-bit uniform, double arithmetic, one rounding.
static inline float wgpt_synth_uniform_at(uint32_t tkey, uint32_t index, double lo, double hi) {
  uint32_t u = wgpt_draw(wgpt_elem_key(tkey, index), 0) >> 8;
  return (float)(lo + (double)u * ((hi - lo) / 16777216.0));
}

#ifdef __cplusplus
}
#endif
#endif  // WGPT_SYNTH_H
