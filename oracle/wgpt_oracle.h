/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the arithmetic of WebGPT's WGSL kernels and of GPT.run().
 * It is the checker for the HIP library and is never linked into, imported by
 * or called from the product path. Only tests, the smoke entry and the
 * cpu_baseline leg of the benchmark may load it.
 *
 * Each function follows one shader of /root/reference (cited per function in
 * wgpt_oracle.c). The shaders cannot be executed where this is built (no WebGPU
 * runtime), so the restatement is pinned by the tests in tests/test_oracle_*.py:
 * float64 numpy brute force, torch CPU library routines, closed forms and the
 * known-answer input of other/test.js:370-388.
 *
 * Choices for what WGSL leaves implementation-defined:
 *   - a*b+sum is evaluated as a multiply then an add (no FMA contraction);
 *   - pow(x,2) and pow(x,3) with a negative base (instructions.js:496,719) are
 *     x*x and x*x*x;
 *   - dot(vec4,vec4) is ((x+y)+z)+w of the four products;
 *   - exp, tanh, sqrt and division are the C library's / IEEE ones.
 */
#ifndef WGPT_ORACLE_H
#define WGPT_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

void ref_set_threads(int n);
int ref_get_threads(void);

/* K1  instructions.js:211-318 (bias may be NULL: K7/K11 add none) */
void ref_matmul_bias(int M, int N, int K, const float* A, const float* B, const float* bias, float* C);
/* K2  instructions.js:358-384 */
void ref_residual(int M, int N, const float* a, const float* b, float* out);
/* K3  instructions.js:451-515: stats[2*row] = mean, stats[2*row+1] = sqrt(var + 1e-5) */
void ref_layernorm_stats(int M, int N, const float* x, float* stats);
/* K4  instructions.js:517-550 */
void ref_layernorm_apply(int M, int N, const float* x, const float* gamma, const float* beta, const float* stats, float* out);
/* K3 + K4, LayerNormBlock.newInstance instructions.js:409-448 */
void ref_layernorm(int M, int N, const float* x, const float* gamma, const float* beta, float* out);
/* K5  instructions.js:593-666 (transpose = false) */
void ref_softmax(int M, int N, const float* x, float* out);
/* K6  instructions.js:705-748 */
void ref_gelu(int M, int N, const float* x, float* out);
/* EmbedBlock.newInstance instructions.js:790-827: out[i] = wte[idx[i]] + wpe[i] */
void ref_embed(const int32_t* idx, int T, int d, const float* wte, const float* wpe, float* out);
/* DeEmbedBlock.newInstance + K7 instructions.js:844-952: logits[V] = x[T-1,:] . wte[v,:] */
void ref_deembed(int d, int V, int T, const float* x, const float* wte, float* logits);
/* K8  instructions.js:1101-1138: [T,d] -> [H,T,hs] */
void ref_format_q(int T, int d, int hs, const float* Q, float* Qf);
/* K9  instructions.js:1141-1178: S[H*T, T] */
void ref_attn_weights(int T, int H, int hs, float scale, const float* Qf, const float* Kmat, float* S);
/* K10 instructions.js:1180-1214: O[T,d] from P[H*T,T], V[T,d] */
void ref_attn_values(int T, int d, int hs, const float* P, const float* V, float* O);
/* AttentionBlock.newFusedInstance instructions.js:985-1099 */
void ref_attention(int T, int d, float scale, int H, int hs, const float* x,
                   const float* Wq, const float* bq, const float* Wk, const float* bk,
                   const float* Wv, const float* bv, const float* Wo, const float* bo, float* out);
/* same, but also hands back K and V ([T,d] each) when non-NULL */
void ref_attention_kv(int T, int d, float scale, int H, int hs, const float* x,
                      const float* Wq, const float* bq, const float* Wk, const float* bk,
                      const float* Wv, const float* bv, const float* Wo, const float* bo, float* out,
                      float* Kout, float* Vout);

/* K11 other/int8-gemm.js:117-229 with a per-column scale (int8-gemm.js:4) */
void ref_dequant_i8(int K, int N, const int32_t* Bq, const float* scale, float* W);
void ref_matmul_i8(int M, int N, int K, const float* A, const int32_t* Bq, const float* scale, const float* bias, float* C);
/* quantizeMatrix other/int8-gemm.js:25-46 (global absmax; returns it) */
float ref_quantize_global(int count, const float* w, int32_t* packed);
/* dequantizeMatrix other/int8-gemm.js:48-62 (double arithmetic, one rounding) */
void ref_dequantize_js(int count, const int32_t* packed, float absmax, float* w);

/* Token selection of GPT.generate, model.js:81-85: selectTopK (globals.js:66-74, stable
 * sort by descending value), cpuSoftmax (globals.js:59-64, float64, temperature inside the
 * exponent), sampleFromDistribution (globals.js:47-57) with `u` for Math.random().
 * ids[k], probs[k] (k = min(top_k, V)) may be NULL. Returns the chosen index. */
int ref_sample_topk(int V, int top_k, double temperature, double u, const float* logits, int32_t* ids, double* probs);

/* Whole model, GPT.run() model.js:104-241. Weight layout is the reference's
 * on-disk one: linear weights [in,out] row-major, c_attn fused [d,3d]. */
typedef struct {
  const float *ln1_g, *ln1_b;
  const float *attn_w, *attn_b;   /* [d,3d], [3d] */
  const float *proj_w, *proj_b;   /* [d,d], [d] */
  const float *ln2_g, *ln2_b;
  const float *fc_w, *fc_b;       /* [d,4d], [4d] */
  const float *fc2_w, *fc2_b;     /* [4d,d], [d] */
  /* int8 variant (NULL for fp32): packed [K,N/4] words + per-column scale */
  const int32_t *attn_q, *proj_q, *fc_q, *fc2_q;
  const float *attn_s, *proj_s, *fc_s, *fc2_s;
} ref_layer;

typedef struct {
  int n_layer, n_head, n_embd, n_ctx, vocab_size;
  const float *wte, *wpe, *lnf_g, *lnf_b;
  const ref_layer* layers;
} ref_model;

/* logits[V] for the last of T tokens. taps (may be NULL) receives
 * (2 + 6*n_layer) arrays of T*d floats in the order tok_pos_emb,
 * block{i}_{ln1,attn,r1,ln2,mlp,r2} ..., ln_f  (other/validation/validation.js:183-205).
 * kv (may be NULL) receives [n_layer][2][T][d]. Returns 0, or -1 on bad arguments. */
int ref_forward(const ref_model* m, const int32_t* tokens, int T, float* logits, float* taps, float* kv);

#ifdef __cplusplus
}
#endif
#endif
