// Launchers of the per-block HIP kernels. All take raw device pointers that the
// caller has already validated against the shapes given; all enqueue on `s`.
#ifndef WGPT_KERNELS_H
#define WGPT_KERNELS_H

#include <hip/hip_runtime.h>
#include <cstdint>

namespace wgpt {

enum Epilogue { EPI_NONE = 0, EPI_GELU = 1, EPI_RESIDUAL = 2 };

// Rows handled per pass of the GEMV path; a matmul with M <= this is a GEMV.
constexpr int GEMV_MAX_ROWS = 4;
constexpr int GEMV_KCHUNK = 64;

// Floats of workspace the GEMV path needs for C[M,N] = A[M,K] . W[K,N].
size_t gemv_workspace_floats(int M, int N, int K);

// C[M,ldc] = epi(A[M,K] . W[K,N] (row stride ldw) + bias) for M <= GEMV_MAX_ROWS.
// bias may be null. resid (EPI_RESIDUAL) has row stride ldc and may alias C.
hipError_t launch_gemv_kn(int M, int N, int K, const float* A, int lda, const float* W, int ldw, const float* bias,
                          float* C, int ldc, int epi, const float* resid, float* workspace, hipStream_t s);

// Same contraction for any M through the tiled GEMM kernels (matrix cores for M >= 16).
// workspace (gemm_workspace_floats(M, N) floats, may be null) enables split-K for
// shapes with too few output tiles to fill the GPU.
size_t gemm_workspace_floats(int M, int N);
// A LayerNormBlock applied to the finished rows of C right after the product (out may not alias C). Where the
// product ends in a split-K reduction pass, that pass normalises the rows it has just finished.
struct LnAfter {
  const float* gamma;
  const float* beta;
  float* out;
  int ldo;
};
// For a product that yields a [M, 3d] q/k/v matrix: the key and value columns of row i also go to row pos0 + i of
// the head-major cache (launch_kv_append's layout), by the pass that finishes C where there is one.
struct KvAfter {
  float* Kc;
  float* Vc;
  int d, hs, ctx, pos0;
};
hipError_t launch_gemm(int M, int N, int K, const float* A, int lda, const float* W, int ldw, const float* bias,
                       float* C, int ldc, int epi, const float* resid, float* workspace, hipStream_t s,
                       const LnAfter* ln = nullptr, const KvAfter* kv = nullptr);
// Same with the packed int8 weights of other/int8-gemm.js (Wq[K, ldwq] words, scale[N]), dequantised inside
// the kernel; M >= 16.
hipError_t launch_gemm_i8(int M, int N, int K, const float* A, int lda, const int32_t* Wq, int ldwq, const float* scale,
                          const float* bias, float* C, int ldc, int epi, const float* resid, float* workspace, hipStream_t s,
                          const LnAfter* ln = nullptr, const KvAfter* kv = nullptr);

// int8 weight-only variants: Wq is [K, ldwq] words holding 4 columns each.
hipError_t launch_gemv_kn_i8(int M, int N, int K, const float* A, int lda, const int32_t* Wq, int ldwq,
                             const float* scale, const float* bias, float* C, int ldc, int epi, const float* resid,
                             float* workspace, hipStream_t s);
hipError_t launch_dequant_i8(int K, int N, const int32_t* Wq, int ldwq, const float* scale, float* W, int ldw, hipStream_t s);

hipError_t launch_residual(size_t n4, const float* a, const float* b, float* out, hipStream_t s);
hipError_t launch_gelu(size_t n4, const float* x, float* out, hipStream_t s);
hipError_t launch_layernorm(int M, int N, const float* x, int ldx, const float* gamma, const float* beta, float* out, int ldo,
                            hipStream_t s);
hipError_t launch_softmax(int M, int N, const float* x, float* out, bool transpose, hipStream_t s);
hipError_t launch_transpose(int rows, int cols, const float* in, float* out, hipStream_t s);
// out[i,:] = wte[idx[i],:] + wpe[pos0+i,:]; idx on the device.
hipError_t launch_embed(const int32_t* idx, int T, int d, int pos0, const float* wte, const float* wpe, float* out, hipStream_t s);
// logits[v] = x . wte[v,:]
hipError_t launch_vocab_gemv(int V, int d, const float* x, const float* wte, float* logits, hipStream_t s);
// Causal attention of Tq query rows (absolute positions pos0..pos0+Tq-1) against
// keys/values 0..pos. q row i is at q + i*ldq + h*hs; key row j of head h is at
// Kc + h*hstride + j*ldkv (likewise values).
hipError_t launch_attention(int Tq, int pos0, int H, int hs, float scale, const float* q, int ldq, const float* Kc,
                            const float* Vc, size_t hstride, int ldkv, float* out, int ldo, hipStream_t s);
// Appends the K and V columns of qkv[T,3d] at positions pos0.. of a head-major cache [H][ctx][hs].
hipError_t launch_kv_append(int T, int d, int hs, int ctx, int pos0, const float* qkv, float* Kc, float* Vc, hipStream_t s);
// Copies rows of src (row stride lds, `cols` floats wide) to dst (row stride ldd).
hipError_t launch_copy_rows(int rows, int cols, const float* src, int lds, float* dst, int ldd, hipStream_t s);
// Top-k / temperature / inverse-CDF selection of one token on the device (globals.js:47-74,
// model.js:81-85); *u is the uniform draw, device memory. tok[0] and out[slot] (optional) get
// the id, ids[k] / probs[k] (optional) the selected indices and their probabilities.
constexpr int SAMPLE_MAX_V = 262144;
constexpr int SAMPLE_MAX_K = 1024;
hipError_t launch_sample_topk(int V, int k, double temperature, const double* u, const float* logits, int32_t* tok,
                              int32_t* out, int slot, int32_t* ids, double* probs, hipStream_t s);
// ---- one decode token with one launch per block; every launch reads the cache position from *pos, so the same
//      launches (recorded once as a HIP graph) serve every token ----
// C[N] = epi(row(x)[K] . W + bias) in one launch and one pass over a decode slab (column c of W is S = ceil(K/256)
// segments of 64 lanes x float4, or x one word of four int8, starting at item c * S). row_mode: GEMV_ROW_PLAIN uses x
// as it is, GEMV_ROW_NORMALISE the LayerNorm of x without gamma and beta (a slab that holds diag(gamma) W, a bias
// that holds bias + beta W), GEMV_ROW_LAYERNORM the LayerNorm with gamma and beta. With kv the key/value columns of
// a q/k/v row also go to cache row *pos.
// With merge (row_mode GEMV_ROW_PLAIN) the row is not x but the attention output that launch_attention_decode_slices
// left in slices, combined while the row is staged.
enum { GEMV_ROW_PLAIN = 0, GEMV_ROW_NORMALISE = 1, GEMV_ROW_LAYERNORM = 2 };
struct AttnSlices {
  float* part;  // [H][nslice][hs + 4]: unnormalised output, then the slice's maximum and sum
  int nslice, hs;
  int nmerge;   // the merge reads the first nmerge slices: at least those that hold positions (nslice is always right)
};
hipError_t launch_gemv_slab(int N, int K, const void* slab, bool int8, const float* scale, const float* x, int row_mode,
                            const float* gamma, const float* beta, const float* bias, float* C, int epi, const float* resid,
                            const KvAfter* kv, const int* pos, hipStream_t s, const AttnSlices* merge = nullptr);
// x[d] = wte[tok[0]] + wpe[*pos]
hipError_t launch_embed_at(const int32_t* tok, int d, const int* pos, const float* wte, const float* wpe, float* x, hipStream_t s);
// Attention of the one query at position *pos (q[h*hs..]) over cache rows 0..*pos of a head-major cache [H][ctx][hs].
hipError_t launch_attention_decode(int H, int hs, int ctx, float scale, const float* q, const float* Kc, const float* Vc, float* out,
                                   const int* pos, hipStream_t s);
// The same for a cache of more than one slice (attention_decode_slices(hs, ctx) > 1; a slice is 4 x 256 / lanes-per-key
// positions, 64 at head size 64): a workgroup per (head, slice), results left in out->part for the merge of
// launch_gemv_slab. spec_pos: the position the caller expects *pos to hold (slices up to it request their rows before
// they have read *pos; any value gives the same results).
int attention_decode_slice_positions(int hs);
int attention_decode_slices(int hs, int ctx);
hipError_t launch_attention_decode_slices(int H, int hs, int ctx, float scale, const float* q, const float* Kc, const float* Vc,
                                          const AttnSlices* out, const int* pos, int spec_pos, hipStream_t s);
// logits[v] = LayerNorm(x) . wte[v,:], then *pos += 1: the end of a decode token.
hipError_t launch_vocab_gemv_ln(int V, int d, const float* x, const float* gamma, const float* beta, const float* wte, float* logits,
                                int* pos, hipStream_t s);

// tok[0] = argmax(logits[0..V)) with the lowest index on ties; also stored to out[slot].
hipError_t launch_argmax(int V, const float* logits, int32_t* tok, int32_t* out, int slot, hipStream_t s);

}  // namespace wgpt

#endif
