/* TEST INFRASTRUCTURE ONLY: CPU restatement of WebGPT's WGSL kernels (see
 * wgpt_oracle.h). Never part of the product path.
 *
 * Build: gcc -O3 -mavx2 -ffp-contract=off -fopenmp -shared -fPIC (oracle/Makefile).
 * -ffp-contract=off keeps a*b+sum as two roundings; loops are arranged so the
 * vectoriser works across independent output elements and never reassociates
 * a sum, so the per-element operation order stays the one the shader has.
 */
#include "wgpt_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0; /* 0 = OpenMP default */

void ref_set_threads(int n) {
  g_threads = n;
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#endif
}

int ref_get_threads(void) {
#ifdef _OPENMP
  return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------------------------------------------------------------------
 * K1 fastMatMul, instructions.js:211-318.
 * Per output element: sum starts at +0, k ascending, sum = a*b + sum
 * (instructions.js:255-301), bias added after the loop (304-314). The shader's
 * 4x8 register tile and its withCheck/noCheck store variants (181-208) do not
 * change any element's arithmetic. N % 8 == 0 is the host's precondition (158);
 * this function accepts any N because K7 reuses it for ragged vocab chunks.
 * ------------------------------------------------------------------------- */
#define MM_ROWS 4
#define MM_COLS 256

static void matmul_tile(int N, int K, const float* A, int lda, const float* B, const float* bias,
                        float* C, int rows, int n0, int ncols) {
  float acc[MM_ROWS][MM_COLS];
  for (int r = 0; r < rows; ++r)
    for (int n = 0; n < ncols; ++n) acc[r][n] = 0.0f;
  for (int k = 0; k < K; ++k) {
    const float* brow = B + (size_t)k * N + n0;
    for (int r = 0; r < rows; ++r) {
      const float a = A[(size_t)r * lda + k];
      float* ar = acc[r];
      for (int n = 0; n < ncols; ++n) ar[n] = a * brow[n] + ar[n];
    }
  }
  for (int r = 0; r < rows; ++r)
    for (int n = 0; n < ncols; ++n)
      C[(size_t)r * N + n0 + n] = bias ? acc[r][n] + bias[n0 + n] : acc[r][n];
}

void ref_matmul_bias(int M, int N, int K, const float* A, const float* B, const float* bias, float* C) {
  const int mt = (M + MM_ROWS - 1) / MM_ROWS;
  const int nt = (N + MM_COLS - 1) / MM_COLS;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int mi = 0; mi < mt; ++mi) {
    for (int ni = 0; ni < nt; ++ni) {
      const int m0 = mi * MM_ROWS, n0 = ni * MM_COLS;
      const int rows = M - m0 < MM_ROWS ? M - m0 : MM_ROWS;
      const int ncols = N - n0 < MM_COLS ? N - n0 : MM_COLS;
      matmul_tile(N, K, A + (size_t)m0 * K, K, B, bias, C + (size_t)m0 * N, rows, n0, ncols);
    }
  }
}

/* K2 elementWiseAddition, instructions.js:381-382 */
void ref_residual(int M, int N, const float* a, const float* b, float* out) {
  const size_t n = (size_t)M * N;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* K3 normStats, instructions.js:451-515. One workgroup of W threads per row,
 * W = 64 unless N > 4096 (instructions.js:412). Thread c sums x[c], x[c+W], ...
 * ascending (473-476); tree: for s = W/2 .. 1: buf[c] += buf[c+s], c < s
 * (481-486); mean = buf[0]/N (489). Variance pass: per-thread sum of squared
 * deviations divided by N before the tree (494-498); stdev = sqrt(v + 1e-5) (508). */
static float tree_sum(float* buf, int W) {
  for (int s = W >> 1; s > 0; s >>= 1)
    for (int c = 0; c < s; ++c) buf[c] = buf[c] + buf[c + s];
  return buf[0];
}

void ref_layernorm_stats(int M, int N, const float* x, float* stats) {
  const int W = N > 4096 ? 256 : 64;
#pragma omp parallel for schedule(static)
  for (int row = 0; row < M; ++row) {
    float buf[256] = {0.0f};
    const float* xr = x + (size_t)row * N;
    for (int c = 0; c < W; ++c) {
      float t = 0.0f;
      for (int i = c; i < N; i += W) t = t + xr[i];
      buf[c] = t;
    }
    const float mean = tree_sum(buf, W) / (float)N;
    for (int c = 0; c < W; ++c) {
      float t = 0.0f;
      for (int i = c; i < N; i += W) {
        const float dlt = xr[i] - mean;
        t = t + dlt * dlt; /* pow(x - mean, 2), instructions.js:496 */
      }
      buf[c] = t / (float)N;
    }
    const float var = tree_sum(buf, W);
    stats[2 * row] = mean;
    stats[2 * row + 1] = sqrtf(var + 1e-5f);
  }
}

/* K4 norm, instructions.js:542-548: gamma * ((x - mean) / stdev) + beta */
void ref_layernorm_apply(int M, int N, const float* x, const float* gamma, const float* beta, const float* stats, float* out) {
#pragma omp parallel for schedule(static)
  for (int row = 0; row < M; ++row) {
    const float mean = stats[2 * row], stdev = stats[2 * row + 1];
    for (int c = 0; c < N; ++c) {
      const float o = (x[(size_t)row * N + c] - mean) / stdev;
      out[(size_t)row * N + c] = gamma[c] * o + beta[c];
    }
  }
}

void ref_layernorm(int M, int N, const float* x, const float* gamma, const float* beta, float* out) {
  float* stats = (float*)malloc(sizeof(float) * 2 * (size_t)M);
  ref_layernorm_stats(M, N, x, stats);
  ref_layernorm_apply(M, N, x, gamma, beta, stats, out);
  free(stats);
}

/* K5 fused softmax, instructions.js:593-666. W = 64 unless N > 4096 (568).
 * max: strided from -3.402823e38 (619-622), combine is order independent;
 * sum: strided exp(x - max) ascending per thread (642-645), full W-wide tree
 * (649-654); out = exp(x - max) / sum (662). */
void ref_softmax(int M, int N, const float* x, float* out) {
  const int W = N > 4096 ? 256 : 64;
#pragma omp parallel for schedule(static)
  for (int row = 0; row < M; ++row) {
    float buf[256] = {0.0f};
    const float* xr = x + (size_t)row * N;
    float mx = -3.402823e+38f;
    for (int i = 0; i < N; ++i) mx = xr[i] > mx ? xr[i] : mx;
    for (int c = 0; c < W; ++c) {
      float t = 0.0f;
      for (int i = c; i < N; i += W) t = t + expf(xr[i] - mx);
      buf[c] = t;
    }
    const float sum = tree_sum(buf, W);
    for (int i = 0; i < N; ++i) out[(size_t)row * N + i] = expf(xr[i] - mx) / sum;
  }
}

/* K6 GELU, instructions.js:711-727 */
void ref_gelu(int M, int N, const float* x, float* out) {
  const size_t n = (size_t)M * N;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) {
    const float v = x[i];
    const float x3 = v * v * v;
    const float cdf = 0.5f * (1.0f + tanhf(0.7978845608f * (v + 0.044715f * x3)));
    float r = v * cdf;
    if (v < -10.0f) r = 0.0f;
    if (v > 10.0f) r = v;
    out[i] = r;
  }
}

/* EmbedBlock, instructions.js:795-821: T row copies out of wte, one slice of
 * wpe starting at position 0, then K2. */
void ref_embed(const int32_t* idx, int T, int d, const float* wte, const float* wpe, float* out) {
  for (int i = 0; i < T; ++i)
    for (int c = 0; c < d; ++c) out[(size_t)i * d + c] = wte[(size_t)idx[i] * d + c] + wpe[(size_t)i * d + c];
}

/* DeEmbedBlock + K7, instructions.js:849-856 (last row only), 916-943 (k
 * ascending, sum = a*b + sum, no bias). The reference multiplies by host-made
 * transposes of zero-padded vocab chunks (model.js:348-364) and concatenates
 * the chunk results (instructions.js:873-880); per logit that is exactly
 * sum_k x[k] * wte[v,k] in ascending k. */
void ref_deembed(int d, int V, int T, const float* x, const float* wte, float* logits) {
  const float* xl = x + (size_t)(T - 1) * d;
#pragma omp parallel for schedule(static)
  for (int v0 = 0; v0 < V; v0 += 8) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    const int nv = V - v0 < 8 ? V - v0 : 8;
    for (int k = 0; k < d; ++k)
      for (int j = 0; j < nv; ++j) acc[j] = xl[k] * wte[(size_t)(v0 + j) * d + k] + acc[j];
    for (int j = 0; j < nv; ++j) logits[v0 + j] = acc[j];
  }
}

/* K8 formatQ, instructions.js:1129-1136 */
void ref_format_q(int T, int d, int hs, const float* Q, float* Qf) {
  for (int r = 0; r < T; ++r)
    for (int c = 0; c < d; ++c) Qf[(size_t)(c / hs) * hs * T + (size_t)r * hs + (c % hs)] = Q[(size_t)r * d + c];
}

/* K9 fusedWeights, instructions.js:1167-1176. Row R = h*T + i. */
void ref_attn_weights(int T, int H, int hs, float scale, const float* Qf, const float* Kmat, float* S) {
  const int d = H * hs;
#pragma omp parallel for schedule(static)
  for (int R = 0; R < H * T; ++R) {
    const int h = R / T, i = R % T;
    const float* q = Qf + (size_t)R * hs;
    for (int j = 0; j < T; ++j) {
      float out = -1e9f;
      if (j <= i) {
        const float* kk = Kmat + (size_t)j * d + (size_t)h * hs;
        float sum = 0.0f;
        for (int k4 = 0; k4 < hs; k4 += 4) {
          const float dot = ((q[k4] * kk[k4] + q[k4 + 1] * kk[k4 + 1]) + q[k4 + 2] * kk[k4 + 2]) + q[k4 + 3] * kk[k4 + 3];
          sum = sum + dot;
        }
        out = sum * scale;
      }
      S[(size_t)R * T + j] = out;
    }
  }
}

/* K10 attentionValues, instructions.js:1205-1212: all j < T ascending, including
 * the masked ones whose weight is exactly 0; sum = sum + v*w. */
void ref_attn_values(int T, int d, int hs, const float* P, const float* V, float* O) {
#pragma omp parallel for schedule(static)
  for (int i = 0; i < T; ++i) {
    float* o = O + (size_t)i * d;
    for (int c = 0; c < d; ++c) o[c] = 0.0f;
    for (int j = 0; j < T; ++j) {
      const float* v = V + (size_t)j * d;
      for (int h = 0; h < d / hs; ++h) {
        const float w = P[(size_t)h * T * T + (size_t)i * T + j];
        for (int c = h * hs; c < (h + 1) * hs; ++c) o[c] = o[c] + v[c] * w;
      }
    }
  }
}

/* AttentionBlock.newFusedInstance, instructions.js:1003-1097:
 * Q,K,V = K1; K8(Q); K9; K5 over [H*T, T]; K10; K1 with the output projection. */
void ref_attention_kv(int T, int d, float scale, int H, int hs, const float* x,
                      const float* Wq, const float* bq, const float* Wk, const float* bk,
                      const float* Wv, const float* bv, const float* Wo, const float* bo, float* out,
                      float* Kout, float* Vout) {
  const size_t td = (size_t)T * d;
  float* Q = (float*)malloc(sizeof(float) * td);
  float* Km = (float*)malloc(sizeof(float) * td);
  float* Vm = (float*)malloc(sizeof(float) * td);
  float* Qf = (float*)malloc(sizeof(float) * td);
  float* S = (float*)malloc(sizeof(float) * (size_t)H * T * T);
  float* P = (float*)malloc(sizeof(float) * (size_t)H * T * T);
  float* O = (float*)malloc(sizeof(float) * td);
  ref_matmul_bias(T, d, d, x, Wq, bq, Q);
  ref_matmul_bias(T, d, d, x, Wk, bk, Km);
  ref_matmul_bias(T, d, d, x, Wv, bv, Vm);
  ref_format_q(T, d, hs, Q, Qf);
  ref_attn_weights(T, H, hs, scale, Qf, Km, S);
  ref_softmax(H * T, T, S, P);
  ref_attn_values(T, d, hs, P, Vm, O);
  ref_matmul_bias(T, d, d, O, Wo, bo, out);
  if (Kout) memcpy(Kout, Km, sizeof(float) * td);
  if (Vout) memcpy(Vout, Vm, sizeof(float) * td);
  free(Q); free(Km); free(Vm); free(Qf); free(S); free(P); free(O);
}

void ref_attention(int T, int d, float scale, int H, int hs, const float* x,
                   const float* Wq, const float* bq, const float* Wk, const float* bk,
                   const float* Wv, const float* bv, const float* Wo, const float* bo, float* out) {
  ref_attention_kv(T, d, scale, H, hs, x, Wq, bq, Wk, bk, Wv, bv, Wo, bo, out, NULL, NULL);
}

/* ---------------------------------------------------------------------------
 * int8 weight-only path, other/int8-gemm.js.
 * Packing (36-43): four consecutive row-major elements per 32-bit word, element
 * 0 in bits 0-7. unpackInt8x4 (126-132): sign extension by (v << 24) >> 24 etc.,
 * element 3 by v >> 24; then f32(b) / 127.0 * scale: two f32 roundings.
 * The sample's single absmax becomes a per-output-column scale (file header,
 * line 4); the sample's max(absmax_A, absmax_B) mix-up (76,124) is not copied.
 * ------------------------------------------------------------------------- */
static inline float dq(int32_t word, int e, float scale) {
  int32_t b;
  if (e == 3) b = word >> 24;
  else b = (int32_t)((uint32_t)word << (24 - 8 * e)) >> 24;
  return (float)b / 127.0f * scale;
}

void ref_dequant_i8(int K, int N, const int32_t* Bq, const float* scale, float* W) {
  const int ND4 = (N + 3) / 4;
#pragma omp parallel for schedule(static)
  for (int k = 0; k < K; ++k)
    for (int n = 0; n < N; ++n) W[(size_t)k * N + n] = dq(Bq[(size_t)k * ND4 + n / 4], n & 3, scale[n]);
}

void ref_matmul_i8(int M, int N, int K, const float* A, const int32_t* Bq, const float* scale, const float* bias, float* C) {
  /* K1's loop with brow = unpackInt8x4(word) (int8-gemm.js:163-209); the
   * dequantised value feeds the same a*b+sum, so dequantise then reuse K1. */
  float* W = (float*)malloc(sizeof(float) * (size_t)K * N);
  ref_dequant_i8(K, N, Bq, scale, W);
  ref_matmul_bias(M, N, K, A, W, bias, C);
  free(W);
}

/* quantizeMatrix, int8-gemm.js:25-46: JS numbers are doubles; Math.round rounds
 * half toward +infinity = floor(x + 0.5); & 0xff keeps the two's complement byte. */
float ref_quantize_global(int count, const float* w, int32_t* packed) {
  double absmax = 0.0;
  for (int i = 0; i < count; ++i) {
    const double a = fabs((double)w[i]);
    if (a > absmax) absmax = a;
  }
  for (int i = 0; i < count; i += 4) {
    uint32_t word = 0;
    for (int e = 0; e < 4; ++e) {
      const double v = i + e < count ? (double)w[i + e] : 0.0;
      const int32_t q = (int32_t)floor((v / absmax) * 127.0 + 0.5);
      word |= ((uint32_t)q & 0xffu) << (8 * e);
    }
    packed[i / 4] = (int32_t)word;
  }
  return (float)absmax;
}

/* dequantizeMatrix, int8-gemm.js:48-62: double arithmetic, one rounding on the
 * store into the Float32Array. May differ from the shader's two roundings by 1 ulp. */
void ref_dequantize_js(int count, const int32_t* packed, float absmax, float* w) {
  for (int i = 0; i < count; ++i) {
    const int32_t word = packed[i / 4];
    const int e = i & 3;
    int32_t b;
    if (e == 3) b = word >> 24;
    else b = (int32_t)((uint32_t)word << (24 - 8 * e)) >> 24;
    w[i] = (float)(((double)b / 127.0) * (double)absmax);
  }
}

/* ---------------------------------------------------------------------------
 * Token selection, model.js:81-85.
 * selectTopK (globals.js:66-74): the (value, index) pairs are sorted with the comparator
 * b.value - a.value; Array.prototype.sort is stable, so equal values keep ascending index.
 * Here: bottom-up merge sort taking from the left run on ties (stable).
 * cpuSoftmax (globals.js:59-64): max over the k values; exp((x - max) / temperature) in
 * float64; sum by reduce from 0, left to right; each term divided by the sum.
 * sampleFromDistribution (globals.js:47-57): running sum, first i with u < sum, else k-1.
 * ------------------------------------------------------------------------- */
int ref_sample_topk(int V, int top_k, double temperature, double u, const float* logits, int32_t* ids, double* probs) {
  int32_t* a = (int32_t*)malloc(sizeof(int32_t) * (size_t)V);
  int32_t* b = (int32_t*)malloc(sizeof(int32_t) * (size_t)V);
  for (int i = 0; i < V; ++i) a[i] = i;
  for (int width = 1; width < V; width *= 2) {
    for (int lo = 0; lo < V; lo += 2 * width) {
      int mid = lo + width < V ? lo + width : V;
      int hi = lo + 2 * width < V ? lo + 2 * width : V;
      int i = lo, j = mid, o = lo;
      while (i < mid && j < hi) {
        /* comparator(left, right) = right.value - left.value > 0 moves right first */
        if (logits[a[j]] > logits[a[i]]) b[o++] = a[j++];
        else b[o++] = a[i++];
      }
      while (i < mid) b[o++] = a[i++];
      while (j < hi) b[o++] = a[j++];
    }
    int32_t* t = a; a = b; b = t;
  }
  const int k = top_k < V ? top_k : V;
  double* e = (double*)malloc(sizeof(double) * (size_t)k);
  double mx = -INFINITY;
  for (int i = 0; i < k; ++i) if ((double)logits[a[i]] > mx) mx = (double)logits[a[i]];
  double sum = 0.0;
  for (int i = 0; i < k; ++i) {
    e[i] = exp(((double)logits[a[i]] - mx) / temperature);
    sum = sum + e[i];
  }
  double cum = 0.0;
  int pick = k - 1, found = 0;
  for (int i = 0; i < k; ++i) {
    const double p = e[i] / sum;
    if (probs) probs[i] = p;
    if (ids) ids[i] = a[i];
    cum += p;
    if (!found && u < cum) { pick = i; found = 1; }
  }
  const int chosen = a[pick];
  free(a); free(b); free(e);
  return chosen;
}

/* ---------------------------------------------------------------------------
 * GPT.run(), model.js:118-240.
 *   r = embed
 *   per layer: a = attention(LN1(r)); r = a + r; m = fc2(gelu(fc(LN2(r)))); r = m + r
 *   logits = deembed(LNf(r))
 * c_attn is split into Q, K, V by columns 0..d, d..2d, 2d..3d
 * (fetchAndSplitQKVWeightTensors model.js:456-468, bias 470-482).
 * ------------------------------------------------------------------------- */
static void split_cols(int K, int N3, int part, const float* W, float* out) {
  const int N = N3 / 3;
  for (int k = 0; k < K; ++k) memcpy(out + (size_t)k * N, W + (size_t)k * N3 + (size_t)part * N, sizeof(float) * N);
}

static void linear(const ref_layer* l, int which, int M, int N, int K, const float* A, float* C) {
  const float* w = which == 1 ? l->proj_w : which == 2 ? l->fc_w : l->fc2_w;
  const float* b = which == 1 ? l->proj_b : which == 2 ? l->fc_b : l->fc2_b;
  const int32_t* q = which == 1 ? l->proj_q : which == 2 ? l->fc_q : l->fc2_q;
  const float* s = which == 1 ? l->proj_s : which == 2 ? l->fc_s : l->fc2_s;
  if (q) ref_matmul_i8(M, N, K, A, q, s, b, C);
  else ref_matmul_bias(M, N, K, A, w, b, C);
}

int ref_forward(const ref_model* m, const int32_t* tokens, int T, float* logits, float* taps, float* kv) {
  const int d = m->n_embd, H = m->n_head, L = m->n_layer, V = m->vocab_size;
  if (T < 1 || T > m->n_ctx || d % 4 || d % H || (d / H) % 4) return -1;
  for (int i = 0; i < T; ++i)
    if (tokens[i] < 0 || tokens[i] >= V) return -1;
  const int hs = d / H, hid = 4 * d;
  const float scale = (float)(1.0 / sqrt((double)hs)); /* model.js:321, uploaded as f32 (instructions.js:1038) */
  const size_t td = (size_t)T * d;
  float* r = (float*)malloc(sizeof(float) * td);
  float* t0 = (float*)malloc(sizeof(float) * td);
  float* t1 = (float*)malloc(sizeof(float) * td);
  float* hbuf = (float*)malloc(sizeof(float) * (size_t)T * hid);
  float* gbuf = (float*)malloc(sizeof(float) * (size_t)T * hid);
  float* wq = (float*)malloc(sizeof(float) * (size_t)d * d);
  float* wk = (float*)malloc(sizeof(float) * (size_t)d * d);
  float* wv = (float*)malloc(sizeof(float) * (size_t)d * d);
  float* wdq = NULL;
  size_t tap = 0;
#define TAP(src) do { if (taps) { memcpy(taps + tap * td, (src), sizeof(float) * td); } ++tap; } while (0)

  ref_embed(tokens, T, d, m->wte, m->wpe, r);
  TAP(r);
  for (int li = 0; li < L; ++li) {
    const ref_layer* l = &m->layers[li];
    ref_layernorm(T, d, r, l->ln1_g, l->ln1_b, t0);
    TAP(t0);
    if (l->attn_q) {
      /* int8 c_attn: dequantise with the shader arithmetic, then the fp32 chain */
      if (!wdq) wdq = (float*)malloc(sizeof(float) * (size_t)d * 3 * d);
      ref_dequant_i8(d, 3 * d, l->attn_q, l->attn_s, wdq);
      split_cols(d, 3 * d, 0, wdq, wq);
      split_cols(d, 3 * d, 1, wdq, wk);
      split_cols(d, 3 * d, 2, wdq, wv);
    } else {
      split_cols(d, 3 * d, 0, l->attn_w, wq);
      split_cols(d, 3 * d, 1, l->attn_w, wk);
      split_cols(d, 3 * d, 2, l->attn_w, wv);
    }
    float* Kout = kv ? kv + ((size_t)li * 2 + 0) * td : NULL;
    float* Vout = kv ? kv + ((size_t)li * 2 + 1) * td : NULL;
    if (l->proj_q) {
      /* output projection is int8 too: run the chain up to K10, then K11 + bias.
       * ref_attention_kv needs an fp32 Wo, so dequantise it (same values). */
      float* wo = (float*)malloc(sizeof(float) * (size_t)d * d);
      ref_dequant_i8(d, d, l->proj_q, l->proj_s, wo);
      ref_attention_kv(T, d, scale, H, hs, t0, wq, l->attn_b, wk, l->attn_b + d, wv, l->attn_b + 2 * d, wo, l->proj_b, t1, Kout, Vout);
      free(wo);
    } else {
      ref_attention_kv(T, d, scale, H, hs, t0, wq, l->attn_b, wk, l->attn_b + d, wv, l->attn_b + 2 * d, l->proj_w, l->proj_b, t1, Kout, Vout);
    }
    TAP(t1);
    ref_residual(T, d, t1, r, r); /* model.js:159 */
    TAP(r);
    ref_layernorm(T, d, r, l->ln2_g, l->ln2_b, t0);
    TAP(t0);
    linear(l, 2, T, hid, d, t0, hbuf);   /* model.js:176 */
    ref_gelu(T, hid, hbuf, gbuf);         /* model.js:188 */
    linear(l, 3, T, d, hid, gbuf, t1);    /* model.js:193 */
    TAP(t1);
    ref_residual(T, d, t1, r, r);         /* model.js:205 */
    TAP(r);
  }
  ref_layernorm(T, d, r, m->lnf_g, m->lnf_b, t0); /* model.js:224 */
  TAP(t0);
  ref_deembed(d, V, T, t0, m->wte, logits);       /* model.js:229 */
#undef TAP
  free(r); free(t0); free(t1); free(hbuf); free(gbuf); free(wq); free(wk); free(wv); free(wdq);
  return 0;
}
