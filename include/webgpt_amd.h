/* webgpt_amd: C ABI of the MI355X (gfx950) implementation of WebGPT's per-token
 * transformer forward path.
 *
 * This is the boundary a host binds (Node N-API addon, ctypes): plain pointers,
 * sizes and integer handles only. Each entry point names the part of the
 * reference (/root/reference, file:line) that it replaces.
 *
 * Conventions
 *   - every function returns 0 on success and a negative code on failure;
 *     wgpt_last_error() then describes the failure (HIP errors are never
 *     swallowed). The reference throws `new Error(msg)` for the same
 *     preconditions (instructions.js:79,158,337,410,684; model.js:294-297);
 *     a host binding turns a non-zero return into a thrown Error.
 *   - all tensors are fp32 row-major; linear weights are [in,out] as in the
 *     reference's weight files. int8 weights are the packing of
 *     other/int8-gemm.js:36-43 (4 consecutive output columns per 32-bit word).
 *   - the library owns all device memory. A wgpt_buf is an opaque handle; the
 *     caller never sees a device pointer. Uploads copy from caller memory and
 *     downloads write into caller memory.
 *   - one HIP stream, not thread-safe: the caller serialises calls, as the
 *     reference's single JS thread and single queue do (model.js:245-263).
 *   - there is no CPU fallback: without a usable gfx950 device every compute
 *     entry point fails.
 */
#ifndef WEBGPT_AMD_H
#define WEBGPT_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef uint64_t wgpt_buf;   /* device buffer handle, 0 = none */
typedef uint64_t wgpt_model; /* model handle, 0 = none */

enum {
  WGPT_OK = 0,
  WGPT_ERR_ARG = -1,     /* precondition violated (shape, alignment, range, size) */
  WGPT_ERR_HIP = -2,     /* a HIP call failed */
  WGPT_ERR_STATE = -3,   /* not initialised, model not finalised, cache overflow */
  WGPT_ERR_NOMEM = -4,
  WGPT_ERR_DEVICE = -5   /* kernel reported a device-side failure (bounded wait expired) */
};

/* ---- lifecycle: navigator.gpu.requestAdapter/requestDevice + initializeOperations
 *      (model.js:25-30, globals.js:13-15); destroyOperations (globals.js:25-27) ---- */
int wgpt_init(int device);
int wgpt_shutdown(void);
const char* wgpt_last_error(void);
/* name: >= 64 bytes. Any out pointer may be NULL. */
int wgpt_device_info(char* name, size_t name_len, int* compute_units, uint64_t* hbm_bytes);

/* ---- buffers: device.createBuffer / mappedAtCreation upload (model.js:490-500,
 *      instructions.js:67-75), copyBufferToBuffer (model.js:254), mapAsync read-back
 *      (model.js:261-263), buffer.destroy (model.js:502-505) ---- */
int wgpt_alloc(size_t bytes, wgpt_buf* out);
int wgpt_free(wgpt_buf buf);
int wgpt_buf_size(wgpt_buf buf, size_t* bytes);
int wgpt_upload(wgpt_buf dst, size_t dst_off, const void* src, size_t bytes);
int wgpt_download(void* dst, wgpt_buf src, size_t src_off, size_t bytes);
int wgpt_copy(wgpt_buf dst, size_t dst_off, wgpt_buf src, size_t src_off, size_t bytes);
int wgpt_sync(void);

/* ---- instruction blocks (instructions.js). Outputs must not alias inputs
 *      unless stated. ---- */

/* FastMatMulBlock.newInstance(rows, cols, shared, in, W, bias) instructions.js:157-177,
 * kernel 211-318: C[M,N] = A[M,K] . W[K,N] + bias[N]. Requires N % 8 == 0 (158)
 * and K % 4 == 0 (vec4 view, 219-220). bias = 0 adds none. */
int wgpt_matmul_bias(int M, int N, int K, wgpt_buf A, wgpt_buf W, wgpt_buf bias, wgpt_buf C);

/* wgpt_matmul_bias for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc, code that runs while another stream of the process is under HIP graph capture; the call itself
 * launches on the library's own stream). It has no counterpart in the reference. Same arithmetic and result as
 * wgpt_matmul_bias for M <= 4 (the batch-1 matrix-vector product), but the ceil(K/64) * M * N partial sums live
 * in a fixed 4 MiB array inside the library's code object (one copy per GPU, held until the process ends)
 * instead of a grow-only hipMalloc: the call allocates and frees nothing. Fails with WGPT_ERR_ARG when M > 4 or
 * when the partial sums exceed 1048576 floats. All calls on a GPU share that array: calls that overlap in time
 * (from several threads or streams) race; the library's single stream orders calls made one after the other. */
int wgpt_matmul_bias_noalloc(int M, int N, int K, wgpt_buf A, wgpt_buf W, wgpt_buf bias, wgpt_buf C);

/* other/int8-gemm.js:117-229 with a per-output-column scale (file header line 4):
 * W[k,n] = float(int8) / 127.0f * scale[n], Wq packed [K, N/4] words. bias = 0 adds none. */
int wgpt_matmul_bias_i8(int M, int N, int K, wgpt_buf A, wgpt_buf Wq, wgpt_buf scale, wgpt_buf bias, wgpt_buf C);
/* unpackInt8x4 other/int8-gemm.js:126-132 applied to a whole matrix: W[K,N] fp32. */
int wgpt_dequant_i8(int K, int N, wgpt_buf Wq, wgpt_buf scale, wgpt_buf W);

/* ResidualBlock.newInstance(rows, cols, a, b) instructions.js:336-384. out may alias a or b. */
int wgpt_residual(int M, int N, wgpt_buf a, wgpt_buf b, wgpt_buf out);
/* LayerNormBlock.newInstance(rows, cols, in, gamma, beta) instructions.js:409-550. */
int wgpt_layernorm(int M, int N, wgpt_buf x, wgpt_buf gamma, wgpt_buf beta, wgpt_buf out);
/* SoftmaxBlock.newInstance(rows, cols, in) instructions.js:567-666. */
int wgpt_softmax(int M, int N, wgpt_buf x, wgpt_buf out);
/* SoftmaxBlock.newInstance(rows, cols, in, transpose = true): the same values stored transposed,
 * out[i * M + row] (instructions.js:594), i.e. out is [N, M]. */
int wgpt_softmax_t(int M, int N, wgpt_buf x, wgpt_buf out);
/* transpose(array, rows, cols) of globals.js:80-94 on the device: out[c * rows + r] = in[r * cols + c].
 * The reference transposes each vocabulary chunk on the host at load time (model.js:362-363); a host that
 * is handed such [d, chunk] buffers turns them back into rows with this. */
int wgpt_transpose(int rows, int cols, wgpt_buf in, wgpt_buf out);
/* GeluBlock.newInstance(rows, cols, in) instructions.js:683-748. out may alias x. */
int wgpt_gelu(int M, int N, wgpt_buf x, wgpt_buf out);
/* EmbedBlock.newInstance(idx, T, d, ...) instructions.js:790-827: out[i] = wte[idx[i]] + wpe[i].
 * idx is a host array of T token ids in [0, V). wte is the whole [V,d] table (the
 * reference's vocab chunking, model.js:298-364, is not needed). */
int wgpt_embed(const int32_t* idx, int T, int d, int V, wgpt_buf wte, wgpt_buf wpe, wgpt_buf out);
/* DeEmbedBlock.newInstance instructions.js:844-952: logits[V] = x[T-1,:] . wte[v,:]. */
int wgpt_deembed(int d, int V, int T, wgpt_buf x, wgpt_buf wte, wgpt_buf logits);
/* AttentionBlock.newFusedInstance instructions.js:985-1214: causal self-attention of
 * x[T,d] including the Q/K/V and output projections. */
int wgpt_attention(int T, int d, float scale, int H, int hs, wgpt_buf x,
                   wgpt_buf Wq, wgpt_buf bq, wgpt_buf Wk, wgpt_buf bk, wgpt_buf Wv, wgpt_buf bv,
                   wgpt_buf Wo, wgpt_buf bo, wgpt_buf out);
/* selectTopK + cpuSoftmax + sampleFromDistribution (globals.js:47-74) over a device
 * buffer of V logits: *id receives the sampled index; ids[top_k] and probs[top_k]
 * (either may be NULL) the selected indices (stable descending order: lowest index
 * first among equal logits) and their float64 probabilities. top_k is clamped to V. */
int wgpt_sample_topk(int V, int top_k, double temperature, double u, wgpt_buf logits, int32_t* id, int32_t* ids,
                     double* probs);

/* ---- whole model: GPT.loadModel + GPT.run (model.js:104-268, 270-488) ---- */
typedef struct {
  int32_t n_layer, n_head, n_embd, n_ctx, vocab_size; /* params_gpt.json, model.js:291-297 */
  int32_t weight_dtype;  /* 0 = fp32 linear weights, 1 = int8 weight-only linear weights */
  int32_t max_prefill;   /* longest prompt accepted by wgpt_prefill; 0 = n_ctx */
  int32_t flags;         /* WGPT_FLAG_* */
} wgpt_params;

enum {
  WGPT_FLAG_TAPS = 1, /* keep the activation taps of the last wgpt_prefill for wgpt_model_tap */
  WGPT_FLAG_TUNE_DELAYS = 2 /* wgpt_model_finalize ends with wgpt_model_tune_poll_delays(m, 2, ...) */
};

int wgpt_model_create(const wgpt_params* params, wgpt_model* out);
/* Tensor names are the reference's weight-file stems (model.js:341,371,379-383,405-420):
 *   transformer.wte.weight [V,d], transformer.wpe.weight [ctx,d],
 *   transformer.ln_f.{weight,bias} [d],
 *   transformer.h.<i>.ln_1.{weight,bias}, .ln_2.{weight,bias} [d],
 *   transformer.h.<i>.attn.c_attn.{weight [d,3d], bias [3d]},
 *   transformer.h.<i>.attn.c_proj.{weight [d,d], bias [d]},
 *   transformer.h.<i>.mlp.c_fc.{weight [d,4d], bias [4d]},
 *   transformer.h.<i>.mlp.c_proj.{weight [4d,d], bias [d]}
 * all fp32. With weight_dtype = 1 the four linear `.weight` tensors are instead
 * given as `<stem>.weight.q` (int32 words [K, N/4]) and `<stem>.weight.scale` (fp32 [N]).
 * The Q/K/V split of c_attn (model.js:456-482) happens inside. data is copied. */
int wgpt_model_set_tensor(wgpt_model m, const char* name, const void* data, size_t bytes);
/* Checks that every tensor arrived and prepares the device-side layouts. */
int wgpt_model_finalize(wgpt_model m);
/* run(idx) for a whole window (model.js:104): resets the KV cache, processes T tokens
 * at positions 0..T-1, writes logits[V] of the last one. logits may be NULL. */
int wgpt_prefill(wgpt_model m, const int32_t* tokens, int T, float* logits);
/* run(idx) for a window that extends the previous one by one token: appends `token`
 * at the next position using the device-resident KV cache. Fails with
 * WGPT_ERR_STATE once n_ctx positions are used (the reference then slides the
 * window and recomputes, model.js:69: the caller does the same with wgpt_prefill). */
int wgpt_decode(wgpt_model m, int32_t token, float* logits);
/* Greedy continuation entirely on the device: starting from `token`, runs `steps`
 * decode steps, each feeding back the arg-max (lowest index on ties, the result of
 * selectTopK with top_k = 1, globals.js:66-74). out_tokens[steps] receives the
 * chosen ids; logits (may be NULL) the logits of the last step. */
int wgpt_decode_greedy(wgpt_model m, int32_t token, int steps, int32_t* out_tokens, float* logits);
/* Sampled continuation on the device: like wgpt_decode_greedy, but each step picks
 * its token the way GPT.generate does (model.js:81-85): selectTopK(logits, top_k),
 * cpuSoftmax(., temperature) in float64 and sampleFromDistribution (globals.js:47-74),
 * with u[i] in [0,1) standing for the i-th Math.random() draw. The V logits never
 * leave the device. top_k in [1, 1024], temperature > 0. */
int wgpt_decode_sample(wgpt_model m, int32_t token, int steps, int top_k, double temperature, const double* u,
                       int32_t* out_tokens, float* logits);
int wgpt_model_reset_cache(wgpt_model m);
int wgpt_model_position(wgpt_model m, int* pos);
/* Activation taps of the last wgpt_prefill (needs WGPT_FLAG_TAPS): names follow
 * other/validation/validation.js:183-205: tok_pos_emb, block<i>_{ln1,attn,r1,ln2,mlp,r2},
 * ln_f (each [T,d]); also kv<i>_k / kv<i>_v: the cache rows 0..pos-1 of layer i ([pos,d]), and, without
 * WGPT_FLAG_TAPS, `residual`: the residual stream after the last layer ([T,d]) of the last wgpt_prefill, which the
 * reference copies into GPT.externalBuffer for its visualisation (model.js:211-222); valid until the next decode. */
int wgpt_model_tap(wgpt_model m, const char* name, float* out, size_t n_floats);
/* GPU time (HIP events on the library's stream) of the last prefill / decode /
 * decode_greedy call, in milliseconds, excluding the logits read-back. */
int wgpt_model_last_gpu_ms(wgpt_model m, float* ms);
/* Algorithmic HBM bytes of one decode step at context length t:
 * weights + 2*L*d*4*t of KV cache. */
int wgpt_model_decode_bytes(wgpt_model m, int t, uint64_t* bytes);
/* Selects the decode implementation: 0 = one kernel per block, 1 = persistent
 * whole-token kernel. Default is the fastest available. */
int wgpt_model_set_decode_mode(wgpt_model m, int mode);
/* The persistent decode kernel waits a fixed time after publishing before it first looks for the other workgroups'
 * values (seven delays, one per exchange; a table per model width is built in, measured on one MI355X). This searches
 * around the current row on the GPU the model lives on: `rounds` passes of coordinate descent (0 = only measure), each
 * candidate timed with multi-step launches at a mid-length context, the found row kept only if it beats the starting
 * one by more than the run-to-run noise when the two are timed alternately. Needs position 0 (before the first
 * prefill, or after wgpt_model_reset_cache); it overwrites key/value rows that every later call rewrites before
 * reading. chosen[7], ms_before, ms_after (milliseconds per token of the starting and the kept row) may be NULL.
 * No counterpart in the reference (its dispatches are ordered by the WebGPU queue). About a second for GPT-2 117M. */
int wgpt_model_tune_poll_delays(wgpt_model m, int rounds, int32_t* chosen, float* ms_before, float* ms_after);
/* The seven delays in use (units of 64 clocks), out[7]. */
int wgpt_model_poll_delays(wgpt_model m, int32_t* out);
int wgpt_model_destroy(wgpt_model m);

/* ---- synthetic tensors (host only, no device needed): the seeded generator the
 *      benchmark configs use in place of the reference's weight files. ---- */
void wgpt_synth_normal(uint32_t seed, uint32_t tensor_id, size_t count, double std_, float* out);
void wgpt_synth_tokens(uint32_t seed, uint32_t tensor_id, size_t count, uint32_t vocab, int32_t* out);
/* packed [K, N/4] words of uniform int8 in [-127,127] */
void wgpt_synth_int8_packed(uint32_t seed, uint32_t tensor_id, size_t K, size_t N, int32_t* out);
void wgpt_synth_uniform(uint32_t seed, uint32_t tensor_id, size_t count, double lo, double hi, float* out);
/* Stable id of a tensor name (FNV-1a of the string), so hosts in any language
 * derive the same tensor_id. */
uint32_t wgpt_synth_tensor_id(const char* name);

#ifdef __cplusplus
}
#endif
#endif /* WEBGPT_AMD_H */
