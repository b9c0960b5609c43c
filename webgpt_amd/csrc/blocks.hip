// C ABI of the instruction blocks: argument validation on the host (shapes against
// buffer sizes, the reference's preconditions with the reference's messages), then
// the kernel launchers of kernels.hip.
#include <cmath>
#include <vector>

#include "common.h"
#include "kernels.h"

namespace wgpt {

// Grow-only device scratch shared by the block entry points (partial sums of the
// GEMV path, the Q/K/V/score temporaries of the attention block, uploaded ids).
struct Scratch {
  void* ptr = nullptr;
  size_t bytes = 0;
};
static Scratch g_scratch[5];

static int grow_scratch(int slot, size_t bytes, void** out) {
  Scratch& s = g_scratch[slot];
  if (s.bytes < bytes) {
    if (s.ptr) {
      WGPT_HIP(hipStreamSynchronize(rt().stream));
      WGPT_HIP(hipFree(s.ptr));
      s.ptr = nullptr;
      s.bytes = 0;
    }
    hipError_t e = hipMalloc(&s.ptr, bytes + 16);
    if (e != hipSuccess) return fail(WGPT_ERR_NOMEM, "hipMalloc(%zu) for scratch: %s", bytes, hipGetErrorString(e));
    s.bytes = bytes;
  }
  *out = s.ptr;
  return WGPT_OK;
}

void release_scratch() {
  for (Scratch& s : g_scratch) {
    if (s.ptr) (void)hipFree(s.ptr);
    s.ptr = nullptr;
    s.bytes = 0;
  }
}

// ---- workspace of the allocation-free matrix-vector entry point (wgpt_matmul_bias_noalloc) ----
// A fixed array in the code object instead of a hipMalloc: NOALLOC_SCRATCH_FLOATS floats (4 MiB) that every GPU
// the library runs on holds until the process ends. In host code the name `scratch` is only a stand-in for the
// symbol, never a device address: the address of this device's copy comes from hipGetSymbolAddress, once per
// device at wgpt_init (setup_noalloc_scratch), and only that pointer is handed to kernels.
constexpr size_t NOALLOC_SCRATCH_FLOATS = (size_t)1 << 20;
static __device__ __align__(256) float scratch[NOALLOC_SCRATCH_FLOATS];
constexpr int NOALLOC_MAX_DEVICES = 64;
static float* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};

int setup_noalloc_scratch(int device) {
  if (device < 0 || device >= NOALLOC_MAX_DEVICES) return fail(WGPT_ERR_ARG, "device %d: no workspace slot (at most %d devices)", device, NOALLOC_MAX_DEVICES);
  if (g_scratch_ptr[device]) return WGPT_OK;
  float* ptr = nullptr;
  hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr)
    return fail(WGPT_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", device, e == hipSuccess ? "null address" : hipGetErrorString(e));
  g_scratch_ptr[device] = ptr;
  return WGPT_OK;
}

static bool overlaps(const void* a, size_t an, const void* b, size_t bn) {
  const char* x = (const char*)a;
  const char* y = (const char*)b;
  return x < y + bn && y < x + an;
}

// Shared by wgpt_matmul_bias and the attention block.
static int matmul_dev(int M, int N, int K, const float* A, const float* W, const float* bias, float* C) {
  hipError_t e;
  if (M <= GEMV_MAX_ROWS) {
    void* ws;
    int rc = grow_scratch(0, sizeof(float) * gemv_workspace_floats(M, N, K), &ws);
    if (rc) return rc;
    e = launch_gemv_kn(M, N, K, A, K, W, N, bias, C, N, EPI_NONE, nullptr, (float*)ws, rt().stream);
  } else {
    void* ws;
    int rc = grow_scratch(0, sizeof(float) * gemm_workspace_floats(M, N), &ws);
    if (rc) return rc;
    e = launch_gemm(M, N, K, A, K, W, N, bias, C, N, EPI_NONE, nullptr, (float*)ws, rt().stream);
  }
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "matmul launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

}  // namespace wgpt

using namespace wgpt;

static inline float* F(wgpt_buf h, size_t count, const char* what) {
  return (float*)resolve(h, sizeof(float) * count, what);
}

extern "C" {

int wgpt_matmul_bias(int M, int N, int K, wgpt_buf A, wgpt_buf W, wgpt_buf bias, wgpt_buf C) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1 || K < 1) return fail(WGPT_ERR_ARG, "wgpt_matmul_bias: M, N, K must be positive");
  if (N % 8 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 16.");  // instructions.js:158
  if (K % 4 != 0) return fail(WGPT_ERR_ARG, "wgpt_matmul_bias: K must be divisible by 4");
  const float* a = F(A, (size_t)M * K, "wgpt_matmul_bias(A)");
  const float* w = F(W, (size_t)K * N, "wgpt_matmul_bias(W)");
  float* c = F(C, (size_t)M * N, "wgpt_matmul_bias(C)");
  if (!a || !w || !c) return WGPT_ERR_ARG;
  const float* b = nullptr;
  if (bias) {
    b = F(bias, N, "wgpt_matmul_bias(bias)");
    if (!b) return WGPT_ERR_ARG;
  }
  if (overlaps(c, sizeof(float) * (size_t)M * N, a, sizeof(float) * (size_t)M * K))
    return fail(WGPT_ERR_ARG, "wgpt_matmul_bias: C must not alias A");
  return matmul_dev(M, N, K, a, w, b, c);
}

int wgpt_matmul_bias_noalloc(int M, int N, int K, wgpt_buf A, wgpt_buf W, wgpt_buf bias, wgpt_buf C) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1 || K < 1) return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_noalloc: M, N, K must be positive");
  if (M > GEMV_MAX_ROWS)
    return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_noalloc: M = %d exceeds the %d rows of the matrix-vector path; use wgpt_matmul_bias", M, GEMV_MAX_ROWS);
  if (N % 8 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 16.");  // instructions.js:158
  if (K % 4 != 0) return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_noalloc: K must be divisible by 4");
  const size_t need = gemv_workspace_floats(M, N, K);
  if (need > NOALLOC_SCRATCH_FLOATS)
    return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_noalloc: ceil(K/%d) * M * N = %zu partial sums exceed the fixed workspace of %zu floats; "
                "use wgpt_matmul_bias", GEMV_KCHUNK, need, NOALLOC_SCRATCH_FLOATS);
  float* ws = rt().device >= 0 && rt().device < NOALLOC_MAX_DEVICES ? g_scratch_ptr[rt().device] : nullptr;
  if (!ws) return fail(WGPT_ERR_STATE, "wgpt_matmul_bias_noalloc: the fixed workspace of device %d was not set up by wgpt_init", rt().device);
  const float* a = F(A, (size_t)M * K, "wgpt_matmul_bias_noalloc(A)");
  const float* w = F(W, (size_t)K * N, "wgpt_matmul_bias_noalloc(W)");
  float* c = F(C, (size_t)M * N, "wgpt_matmul_bias_noalloc(C)");
  if (!a || !w || !c) return WGPT_ERR_ARG;
  const float* b = nullptr;
  if (bias) {
    b = F(bias, N, "wgpt_matmul_bias_noalloc(bias)");
    if (!b) return WGPT_ERR_ARG;
  }
  if (overlaps(c, sizeof(float) * (size_t)M * N, a, sizeof(float) * (size_t)M * K))
    return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_noalloc: C must not alias A");
  // Nothing of the workspace has to start at zero: the first kernel writes every partial sum the second one reads.
  hipError_t e = launch_gemv_kn(M, N, K, a, K, w, N, b, c, N, EPI_NONE, nullptr, ws, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "matmul launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_matmul_bias_i8(int M, int N, int K, wgpt_buf A, wgpt_buf Wq, wgpt_buf scale, wgpt_buf bias, wgpt_buf C) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1 || K < 1) return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_i8: M, N, K must be positive");
  if (N % 8 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 16.");
  if (K % 4 != 0) return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_i8: K must be divisible by 4");
  const float* a = F(A, (size_t)M * K, "wgpt_matmul_bias_i8(A)");
  const int32_t* wq = (const int32_t*)resolve(Wq, sizeof(int32_t) * (size_t)K * (N / 4), "wgpt_matmul_bias_i8(Wq)");
  const float* sc = F(scale, N, "wgpt_matmul_bias_i8(scale)");
  float* c = F(C, (size_t)M * N, "wgpt_matmul_bias_i8(C)");
  if (!a || !wq || !sc || !c) return WGPT_ERR_ARG;
  const float* b = nullptr;
  if (bias) {
    b = F(bias, N, "wgpt_matmul_bias_i8(bias)");
    if (!b) return WGPT_ERR_ARG;
  }
  if (overlaps(c, sizeof(float) * (size_t)M * N, a, sizeof(float) * (size_t)M * K))
    return fail(WGPT_ERR_ARG, "wgpt_matmul_bias_i8: C must not alias A");
  hipError_t e;
  if (M <= GEMV_MAX_ROWS) {
    void* ws;
    int rc = grow_scratch(0, sizeof(float) * gemv_workspace_floats(M, N, K), &ws);
    if (rc) return rc;
    e = launch_gemv_kn_i8(M, N, K, a, K, wq, N / 4, sc, b, c, N, EPI_NONE, nullptr, (float*)ws, rt().stream);
  } else if (M >= 16) {
    // Dense contraction on the matrix cores, words dequantised on their way into LDS (same arithmetic).
    void* ws;
    int rc = grow_scratch(0, sizeof(float) * gemm_workspace_floats(M, N), &ws);
    if (rc) return rc;
    e = launch_gemm_i8(M, N, K, a, K, wq, N / 4, sc, b, c, N, EPI_NONE, nullptr, (float*)ws, rt().stream);
  } else {
    // A few rows more than the matrix-vector kernel takes: dequantise once (same arithmetic), then the fp32 tile kernel.
    void* wf;
    int rc = grow_scratch(1, sizeof(float) * (size_t)K * N, &wf);
    if (rc) return rc;
    e = launch_dequant_i8(K, N, wq, N / 4, sc, (float*)wf, N, rt().stream);
    if (e == hipSuccess) e = launch_gemm(M, N, K, a, K, (const float*)wf, N, b, c, N, EPI_NONE, nullptr, nullptr, rt().stream);
  }
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "int8 matmul launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_dequant_i8(int K, int N, wgpt_buf Wq, wgpt_buf scale, wgpt_buf W) {
  WGPT_REQUIRE_INIT();
  if (K < 1 || N < 1 || N % 4 != 0) return fail(WGPT_ERR_ARG, "wgpt_dequant_i8: K >= 1 and N a positive multiple of 4 required");
  const int32_t* wq = (const int32_t*)resolve(Wq, sizeof(int32_t) * (size_t)K * (N / 4), "wgpt_dequant_i8(Wq)");
  const float* sc = F(scale, N, "wgpt_dequant_i8(scale)");
  float* w = F(W, (size_t)K * N, "wgpt_dequant_i8(W)");
  if (!wq || !sc || !w) return WGPT_ERR_ARG;
  hipError_t e = launch_dequant_i8(K, N, wq, N / 4, sc, w, N, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "dequant launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_residual(int M, int N, wgpt_buf a, wgpt_buf b, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1) return fail(WGPT_ERR_ARG, "wgpt_residual: M and N must be positive");
  if (N % 4 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 4.");  // instructions.js:337
  const size_t n = (size_t)M * N;
  const float* pa = F(a, n, "wgpt_residual(a)");
  const float* pb = F(b, n, "wgpt_residual(b)");
  float* po = F(out, n, "wgpt_residual(out)");
  if (!pa || !pb || !po) return WGPT_ERR_ARG;
  hipError_t e = launch_residual(n / 4, pa, pb, po, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "residual launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_layernorm(int M, int N, wgpt_buf x, wgpt_buf gamma, wgpt_buf beta, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1) return fail(WGPT_ERR_ARG, "wgpt_layernorm: M and N must be positive");
  if (N % 4 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 4.");  // instructions.js:410
  const size_t n = (size_t)M * N;
  const float* px = F(x, n, "wgpt_layernorm(x)");
  const float* pg = F(gamma, N, "wgpt_layernorm(gamma)");
  const float* pb = F(beta, N, "wgpt_layernorm(beta)");
  float* po = F(out, n, "wgpt_layernorm(out)");
  if (!px || !pg || !pb || !po) return WGPT_ERR_ARG;
  if (px == po) return fail(WGPT_ERR_ARG, "wgpt_layernorm: out must not alias x");
  hipError_t e = launch_layernorm(M, N, px, N, pg, pb, po, N, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "layernorm launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_softmax(int M, int N, wgpt_buf x, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1) return fail(WGPT_ERR_ARG, "wgpt_softmax: M and N must be positive");
  const size_t n = (size_t)M * N;
  const float* px = F(x, n, "wgpt_softmax(x)");
  float* po = F(out, n, "wgpt_softmax(out)");
  if (!px || !po) return WGPT_ERR_ARG;
  if (px == po) return fail(WGPT_ERR_ARG, "wgpt_softmax: out must not alias x");
  hipError_t e = launch_softmax(M, N, px, po, false, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "softmax launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_softmax_t(int M, int N, wgpt_buf x, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1) return fail(WGPT_ERR_ARG, "wgpt_softmax_t: M and N must be positive");
  const size_t n = (size_t)M * N;
  const float* px = F(x, n, "wgpt_softmax_t(x)");
  float* po = F(out, n, "wgpt_softmax_t(out)");
  if (!px || !po) return WGPT_ERR_ARG;
  if (px == po) return fail(WGPT_ERR_ARG, "wgpt_softmax_t: out must not alias x");
  hipError_t e = launch_softmax(M, N, px, po, true, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "softmax launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_transpose(int rows, int cols, wgpt_buf in, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (rows < 1 || cols < 1) return fail(WGPT_ERR_ARG, "wgpt_transpose: rows and cols must be positive");
  const size_t n = (size_t)rows * cols;
  const float* pi = F(in, n, "wgpt_transpose(in)");
  float* po = F(out, n, "wgpt_transpose(out)");
  if (!pi || !po) return WGPT_ERR_ARG;
  if (pi == po) return fail(WGPT_ERR_ARG, "wgpt_transpose: out must not alias in");
  hipError_t e = launch_transpose(rows, cols, pi, po, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "transpose launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_sample_topk(int V, int top_k, double temperature, double u, wgpt_buf logits, int32_t* id, int32_t* ids,
                     double* probs) {
  WGPT_REQUIRE_INIT();
  if (V < 1 || V > SAMPLE_MAX_V) return fail(WGPT_ERR_ARG, "wgpt_sample_topk: V must be in [1, %d]", SAMPLE_MAX_V);
  if (top_k < 1 || top_k > SAMPLE_MAX_K) return fail(WGPT_ERR_ARG, "wgpt_sample_topk: top_k must be in [1, %d]", SAMPLE_MAX_K);
  if (!(temperature > 0.0)) return fail(WGPT_ERR_ARG, "wgpt_sample_topk: temperature must be positive");
  if (!(u >= 0.0 && u < 1.0)) return fail(WGPT_ERR_ARG, "wgpt_sample_topk: u must be in [0, 1)");
  if (!id) return fail(WGPT_ERR_ARG, "wgpt_sample_topk: id is NULL");
  const float* pl = F(logits, (size_t)V, "wgpt_sample_topk(logits)");
  if (!pl) return WGPT_ERR_ARG;
  const int k = top_k < V ? top_k : V;
  // scratch: [u | probs[k]] doubles, then [tok | ids[k]] ints
  void* ws;
  int rc = grow_scratch(4, sizeof(double) * (size_t)(1 + k) + sizeof(int32_t) * (size_t)(1 + k), &ws);
  if (rc) return rc;
  double* du = (double*)ws;
  double* dprobs = du + 1;
  int32_t* dtok = (int32_t*)(dprobs + k);
  int32_t* dids = dtok + 1;
  WGPT_HIP(hipMemcpyAsync(du, &u, sizeof(double), hipMemcpyHostToDevice, rt().stream));
  hipError_t e = launch_sample_topk(V, k, temperature, du, pl, dtok, nullptr, 0, dids, dprobs, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "sample_topk launch: %s", hipGetErrorString(e));
  WGPT_HIP(hipMemcpyAsync(id, dtok, sizeof(int32_t), hipMemcpyDeviceToHost, rt().stream));
  if (ids) WGPT_HIP(hipMemcpyAsync(ids, dids, sizeof(int32_t) * (size_t)k, hipMemcpyDeviceToHost, rt().stream));
  if (probs) WGPT_HIP(hipMemcpyAsync(probs, dprobs, sizeof(double) * (size_t)k, hipMemcpyDeviceToHost, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  return WGPT_OK;
}

int wgpt_gelu(int M, int N, wgpt_buf x, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (M < 1 || N < 1) return fail(WGPT_ERR_ARG, "wgpt_gelu: M and N must be positive");
  if (N % 4 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 4.");  // instructions.js:684
  const size_t n = (size_t)M * N;
  const float* px = F(x, n, "wgpt_gelu(x)");
  float* po = F(out, n, "wgpt_gelu(out)");
  if (!px || !po) return WGPT_ERR_ARG;
  hipError_t e = launch_gelu(n / 4, px, po, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "gelu launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_embed(const int32_t* idx, int T, int d, int V, wgpt_buf wte, wgpt_buf wpe, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (!idx || T < 1 || d < 4 || V < 1) return fail(WGPT_ERR_ARG, "wgpt_embed: idx, T >= 1, d >= 4 and V >= 1 required");
  if (d % 4 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 4.");
  for (int i = 0; i < T; ++i)
    if (idx[i] < 0 || idx[i] >= V) return fail(WGPT_ERR_ARG, "wgpt_embed: token id %d at %d outside [0, %d)", idx[i], i, V);
  const float* pe = F(wte, (size_t)V * d, "wgpt_embed(wte)");
  const float* pp = F(wpe, (size_t)T * d, "wgpt_embed(wpe)");
  float* po = F(out, (size_t)T * d, "wgpt_embed(out)");
  if (!pe || !pp || !po) return WGPT_ERR_ARG;
  void* didx;
  int rc = grow_scratch(2, sizeof(int32_t) * (size_t)T, &didx);
  if (rc) return rc;
  WGPT_HIP(hipMemcpyAsync(didx, idx, sizeof(int32_t) * (size_t)T, hipMemcpyHostToDevice, rt().stream));
  // idx is caller memory that may change once this returns: finish the copy first.
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  hipError_t e = launch_embed((const int32_t*)didx, T, d, 0, pe, pp, po, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "embed launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_deembed(int d, int V, int T, wgpt_buf x, wgpt_buf wte, wgpt_buf logits) {
  WGPT_REQUIRE_INIT();
  if (d < 4 || d % 4 != 0 || V < 1 || T < 1) return fail(WGPT_ERR_ARG, "wgpt_deembed: d a positive multiple of 4, V >= 1, T >= 1 required");
  if (d > 12288) return fail(WGPT_ERR_ARG, "wgpt_deembed: d above 12288 is not supported");
  const float* px = F(x, (size_t)T * d, "wgpt_deembed(x)");
  const float* pe = F(wte, (size_t)V * d, "wgpt_deembed(wte)");
  float* pl = F(logits, V, "wgpt_deembed(logits)");
  if (!px || !pe || !pl) return WGPT_ERR_ARG;
  hipError_t e = launch_vocab_gemv(V, d, px + (size_t)(T - 1) * d, pe, pl, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "deembed launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

int wgpt_attention(int T, int d, float scale, int H, int hs, wgpt_buf x, wgpt_buf Wq, wgpt_buf bq, wgpt_buf Wk,
                   wgpt_buf bk, wgpt_buf Wv, wgpt_buf bv, wgpt_buf Wo, wgpt_buf bo, wgpt_buf out) {
  WGPT_REQUIRE_INIT();
  if (T < 1 || d < 8 || H < 1 || hs < 4) return fail(WGPT_ERR_ARG, "wgpt_attention: T, d, H, hs must be positive");
  if (H * hs != d) return fail(WGPT_ERR_ARG, "wgpt_attention: n_head * head_size must equal n_embd");
  if (d % 8 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 16.");
  if (hs % 4 != 0 || hs > 256) return fail(WGPT_ERR_ARG, "wgpt_attention: head_size must be a multiple of 4, at most 256");
  if (T > 12288) return fail(WGPT_ERR_ARG, "wgpt_attention: T above 12288 is not supported");
  const size_t td = (size_t)T * d, dd = (size_t)d * d;
  const float* px = F(x, td, "wgpt_attention(x)");
  const float* wq = F(Wq, dd, "wgpt_attention(Wq)");
  const float* wk = F(Wk, dd, "wgpt_attention(Wk)");
  const float* wv = F(Wv, dd, "wgpt_attention(Wv)");
  const float* wo = F(Wo, dd, "wgpt_attention(Wo)");
  const float* pbq = F(bq, d, "wgpt_attention(bq)");
  const float* pbk = F(bk, d, "wgpt_attention(bk)");
  const float* pbv = F(bv, d, "wgpt_attention(bv)");
  const float* pbo = F(bo, d, "wgpt_attention(bo)");
  float* po = F(out, td, "wgpt_attention(out)");
  if (!px || !wq || !wk || !wv || !wo || !pbq || !pbk || !pbv || !pbo || !po) return WGPT_ERR_ARG;
  if (px == po) return fail(WGPT_ERR_ARG, "wgpt_attention: out must not alias x");
  void* tmp;
  int rc = grow_scratch(3, sizeof(float) * 4 * td, &tmp);
  if (rc) return rc;
  float* Q = (float*)tmp;
  float* Km = Q + td;
  float* Vm = Km + td;
  float* O = Vm + td;
  if ((rc = matmul_dev(T, d, d, px, wq, pbq, Q))) return rc;
  if ((rc = matmul_dev(T, d, d, px, wk, pbk, Km))) return rc;
  if ((rc = matmul_dev(T, d, d, px, wv, pbv, Vm))) return rc;
  hipError_t e = launch_attention(T, 0, H, hs, scale, Q, d, Km, Vm, (size_t)hs, d, O, d, rt().stream);
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "attention launch: %s", hipGetErrorString(e));
  return matmul_dev(T, d, d, O, wo, pbo, po);
}

}  // extern "C"
