// Host interface of the whole-token persistent decode kernel.
#ifndef WGPT_DECODE_PERSISTENT_H
#define WGPT_DECODE_PERSISTENT_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace wgpt {

constexpr int PD_THREADS = 512;  // threads per workgroup
constexpr int PD_GRID = 256;     // workgroups: one per compute unit of an MI355X
constexpr int PD_SPLIT = 4;      // position slices per head in the attention phase (contexts up to PD_SHORT_KEYS)
constexpr int PD_SPLIT_LONG = 8; // ... beyond
constexpr int PD_TOPK = 8;       // largest top_k the kernel samples from itself
constexpr int PD_COLP = 256;     // floats of one workgroup's column parameters of a layer (4 phases x 32 columns x {bias, scale})
constexpr int PD_KVBATCH = 4;    // key batches (of 32) a slice holds in registers: n_ctx <= 32*PD_KVBATCH*PD_SPLIT_LONG
constexpr int PD_SHORT_KEYS = 32 * PD_KVBATCH * PD_SPLIT;  // longest context of the instantiation with PD_SPLIT slices
constexpr int PD_NARROW_D = 1024;  // widest fp32 shape with LDS and registers to spare (table rows kept on the chip, host logits)
constexpr int PD_TABLE_LDS_STEPS = 2;  // launches of at least this many steps keep part of the vocabulary table in LDS

// How one linear layer is split over the workgroups: workgroup w finishes columns
// [w*cpw, (w+1)*cpw) of N; a column is S segments ("items") of 256 contraction elements,
// stored column by column.
struct PhaseGeom {
  int N, cpw, S;
};

// Offsets (in floats) inside one layer's block of small parameters:
// [c_attn bias 3d | attn c_proj bias d | c_fc bias 4d | mlp c_proj bias d | ln1 g,b | ln2 g,b |
//  int8 scales of the four matrices 3d, d, 4d, d].
struct LayerParamOffsets {
  int bA, bC, bD, bE, ln1g, ln1b, ln2g, ln2b;
  int sA, sC, sD, sE;  // per-column scales of the int8 variant; for fp32 weights sA and sD hold the column sums of diag(gamma) W
  // int8 variant, the two matrices behind a LayerNorm: gA, gD the column sums sum_k gamma_k q_kn of the quantised
  // weights, fA, fD the biases with the LayerNorm's beta folded in, bias_n + scale_n / 127 sum_k beta_k q_kn (fold_ln_i8)
  int gA, gD, fA, fD;
  int stride;
};
__host__ __device__ inline LayerParamOffsets layer_param_offsets(int d) {
  LayerParamOffsets o;
  o.bA = 0; o.bC = 3 * d; o.bD = 4 * d; o.bE = 8 * d;
  o.ln1g = 9 * d; o.ln1b = 10 * d; o.ln2g = 11 * d; o.ln2b = 12 * d;
  o.sA = 13 * d; o.sC = 16 * d; o.sD = 17 * d; o.sE = 21 * d;
  o.gA = 22 * d; o.gD = 25 * d; o.fA = 29 * d; o.fD = 32 * d;
  o.stride = 36 * d;
  return o;
}

struct PersistentArgs {
  int L, H, d, ctx, V;
  float scale;
  int rows_per_wg;  // vocabulary rows per workgroup
  int weight_dtype;  // 0: fp32 items (float4 per lane), 1: int8 items (one word per lane)
  // slab-layout weights of all layers in one allocation: layer l starts at
  // slabs + l*slab_stride; c_attn at 0, then attn c_proj, c_fc, mlp c_proj (item-lane units)
  const void* slabs;
  size_t slab_stride, slab_offC, slab_offD, slab_offE;
  const float* lparams;  // [L][36d] small per-layer parameters (LayerParamOffsets)
  const float* colparams;  // [L][PD_GRID][PD_COLP] biases and int8 scales / 127 per workgroup (build_colparams)
  const float *wte, *wpe, *lnf_g, *lnf_b;
  float* kv;  // [L][2][H][ctx][hs]
  // {value, epoch} exchange buffers
  unsigned long long *bufQKV, *bufATT, *bufR1, *bufH, *bufR2, *bufAM;
  float* logits;
  const int32_t* tok;  // tok[0]: token of the first step; null: tok_value is (a call that brings its token as an argument saves a copy)
  int32_t tok_value;
  int32_t* out_tok;    // [nsteps] arg-max of each step
  int* err;            // set non-zero when a bounded wait expired
  unsigned long long* trace;  // optional [G][512] clock samples of the last step (WGPT_TRACE builds), or null
  // naps (about 64 clocks each) between a publish and the first poll of the words that
  // follow it: [0] residual row into c_attn, [1] q/k/v into the attention slices,
  // [2] attention outputs on the attention workgroups, [3] on the others,
  // [4] residual row into c_fc, [5] hidden row, [6] arg-max candidates
  int delay[7];
  // the attention slices take longer the longer the context: delay[2] and delay[3] grow by att_slope[0] and
  // att_slope[1] units per 1024 positions of the step's context
  int att_slope[2];
  unsigned spin_limit;  // poll rounds after which a wait gives up and raises *err
  int short_keys;       // a launch whose last step attends to more positions runs the instantiation with PD_SPLIT_LONG slices (<= PD_SHORT_KEYS)
  // token selection: top_k == 1 is the arg-max; 2..PD_TOPK samples as GPT.generate does
  // (model.js:81-85) with u[step] for the step's Math.random() and the float64 temperature
  int top_k;
  double temperature;
  const double* u;  // [nsteps], device memory (unused for top_k == 1)
  unsigned ebase;      // epoch of the last word published by earlier launches
  int pos0, nsteps;
  // Results written straight into pinned host memory, so that a call of one step needs no copy behind the kernel
  // (both may be null). host_logits[V]: the logits of the last step (shapes persistent_writes_host_logits names;
  // needs rows_per_wg <= 4 d). host_done: workgroup 0 stores *err there once it has finished the last step, which
  // it can only after every workgroup has published its last word; a launch that gave up leaves the word alone.
  float* host_logits;
  int* host_done;
};

PhaseGeom make_geom(int N, int K);
size_t slab_float4s(const PhaseGeom& g);
// Re-lays W[K, N] (row stride ldw) into the slab layout of geometry g; with rowscale
// (the gamma of the LayerNorm in front of the matrix, or null) as diag(rowscale) W.
hipError_t build_slab(const float* W, int ldw, int K, const PhaseGeom& g, const float* rowscale, float4* slab, hipStream_t s);
// out[N] = bias + beta W: the beta of that LayerNorm folded into the bias; colsum[N] = column sums of diag(gamma) W.
// The same for packed int8 weights (Wq[K, N/4] words, scale[N]; other/int8-gemm.js:36-43), whose gamma cannot be folded
// into the quantised values: out_bias[n] = bias[n] + scale[n] / 127 sum_k beta[k] q[k][n], gsum[n] = sum_k gamma[k] q[k][n]
// (both accumulated in double, rounded once).
hipError_t fold_ln_i8(const int32_t* Wq, int ldwq, int K, int N, const float* scale, const float* gamma, const float* beta,
                      const float* bias, float* out_bias, float* gsum, hipStream_t s);
hipError_t fold_ln_bias(const float* W, int ldw, int K, int N, const float* gamma, const float* beta, const float* bias, float* out,
                        float* colsum, hipStream_t s);
// Same for int8 words Wq[K, ldwq] (4 columns per word): one word per item lane.
hipError_t build_slab_i8(const int32_t* Wq, int ldwq, int K, const PhaseGeom& g, int32_t* slab, hipStream_t s);
// Biases and (int8) column scales / 127 of lparams re-laid per layer and workgroup: float t of a block is
// parameter kind t / 128 (bias, scale) of local column t % 32 of linear phase (t / 32) % 4, zero where the
// workgroup has no such column.
hipError_t build_colparams(const float* lparams, int L, int d, int weight_dtype, float* out, hipStream_t s);
// Model shapes the persistent kernel is instantiated for.
bool persistent_supports(int d, int n_head, int n_ctx, int weight_dtype);
// Shapes whose kernel can write the last step's logits to host memory itself (PersistentArgs::host_logits).
bool persistent_writes_host_logits(int d, int weight_dtype);
// Epochs consumed by one decode step.
inline unsigned persistent_epochs_per_step(int L) { return 5u * (unsigned)L + 1u; }
hipError_t launch_decode_persistent(const PersistentArgs& a, hipStream_t s);

}  // namespace wgpt

#endif
