// Per-block HIP kernels for gfx950 (wave64). One kernel family per instruction
// block of the reference (instructions.js); the arithmetic each one reproduces is
// cited at the kernel. Summation orders differ from the WGSL (lanes split the
// reduction and combine by wave shuffles), which stays inside the fp32 tolerance.
#include "kernels.h"

#include <type_traits>

namespace wgpt {

namespace {

constexpr int WG = 256;     // threads per workgroup for every kernel here
constexpr int NWAVE = WG / 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// Sum over a 256-thread workgroup; `sh` holds NWAVE floats. Every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float* sh) {
  v = wave_sum(v);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  v = (sh[0] + sh[1]) + (sh[2] + sh[3]);
  __syncthreads();
  return v;
}

__device__ __forceinline__ float block_max(float v, float* sh) {
  v = wave_max(v);
  if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
  __syncthreads();
  v = fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
  __syncthreads();
  return v;
}

// GELU of the reference, instructions.js:718-727: tanh form, exact 0 below -10,
// identity above 10; x^3 as x*x*x.
__device__ __forceinline__ float gelu_ref(float x) {
  const float x3 = x * x * x;
  const float cdf = 0.5f * (1.0f + tanhf(0.7978845608f * (x + 0.044715f * x3)));
  float r = x * cdf;
  r = x < -10.0f ? 0.0f : r;
  r = x > 10.0f ? x : r;
  return r;
}

// The same for a slab word, whose four bytes are consecutive k of ONE column (scale in every component of sc).
__device__ __forceinline__ float4 unpack_i8x4_k(int32_t word, const float4& sc);

__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }

__device__ __forceinline__ void fma4(float4& acc, float a, const float4& w) {
  acc.x += a * w.x;
  acc.y += a * w.y;
  acc.z += a * w.z;
  acc.w += a * w.w;
}

// unpackInt8x4, other/int8-gemm.js:126-132: sign-extend each byte, then
// f32(b) / 127.0 * scale with a rounding after the divide and after the multiply.
__device__ __forceinline__ float4 unpack_i8x4(int32_t word, const float4& sc) {
  const int b0 = (word << 24) >> 24;
  const int b1 = (word << 16) >> 24;
  const int b2 = (word << 8) >> 24;
  const int b3 = word >> 24;
  float4 r;
  r.x = __fdiv_rn((float)b0, 127.0f) * sc.x;
  r.y = __fdiv_rn((float)b1, 127.0f) * sc.y;
  r.z = __fdiv_rn((float)b2, 127.0f) * sc.z;
  r.w = __fdiv_rn((float)b3, 127.0f) * sc.w;
  return r;
}
__device__ __forceinline__ float4 unpack_i8x4_k(int32_t word, const float4& sc) { return unpack_i8x4(word, sc); }

// ---------------------------------------------------------------------------
// FastMatMulBlock for M <= 4 (batch-1 decode): C = A . W + bias,
// instructions.js:248-314. W is [K,N] row-major as the reference keeps it.
// Stage 1: a workgroup owns a 64-column x 64-row tile of W; 16 lanes read one
// 256-byte row segment as float4s, the 16 lane groups take rows k0+ty, +16, ...
// and combine through LDS. Stage 2 sums the K/64 partials in ascending order,
// adds the bias last (as the shader does) and applies the epilogue.
// ---------------------------------------------------------------------------
template <int R>
__global__ __launch_bounds__(WG) void gemv_kn_partial(int N, int K, const float* __restrict__ A, int lda,
                                                       const float* __restrict__ W, int ldw, float* __restrict__ part) {
  __shared__ float4 red[R][16][16];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int n0 = blockIdx.x * 64 + tx * 4;
  const int k0 = blockIdx.y * GEMV_KCHUNK;
  float4 acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
  if (n0 < N) {
#pragma unroll
    for (int i = 0; i < GEMV_KCHUNK / 16; ++i) {
      const int k = k0 + ty + 16 * i;
      if (k < K) {
        const float4 w = ld4(W + (size_t)k * ldw + n0);
#pragma unroll
        for (int r = 0; r < R; ++r) fma4(acc[r], A[(size_t)r * lda + k], w);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) red[r][ty][tx] = acc[r];
  __syncthreads();
  if (ty < R && n0 < N) {
    float4 s = red[ty][0][tx];
#pragma unroll
    for (int j = 1; j < 16; ++j) {
      const float4 v = red[ty][j][tx];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    st4(part + ((size_t)blockIdx.y * R + ty) * N + n0, s);
  }
}

// With kv.Kc set, C is a [M, 3d] q/k/v matrix whose key and value columns also go to the head-major cache
// (kv_append_kernel's layout).
__global__ __launch_bounds__(WG) void gemv_reduce(int M, int N, int S, const float* __restrict__ part,
                                                   const float* __restrict__ bias, float* C, int ldc, int epi,
                                                   const float* resid, KvAfter kv = KvAfter{nullptr, nullptr, 0, 0, 0, 0}) {
  const int n4 = N >> 2;
  const int idx = blockIdx.x * WG + threadIdx.x;
  if (idx >= M * n4) return;
  const int r = idx / n4, n0 = (idx - r * n4) * 4;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int sp = 0; sp < S; ++sp) {
    const float4 v = ld4(part + ((size_t)sp * M + r) * N + n0);
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  if (bias) {
    const float4 b = ld4(bias + n0);
    s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
  }
  if (epi == EPI_GELU) {
    s.x = gelu_ref(s.x); s.y = gelu_ref(s.y); s.z = gelu_ref(s.z); s.w = gelu_ref(s.w);
  } else if (epi == EPI_RESIDUAL) {
    const float4 q = ld4(resid + (size_t)r * ldc + n0);
    s.x += q.x; s.y += q.y; s.z += q.z; s.w += q.w;
  }
  st4(C + (size_t)r * ldc + n0, s);
  if (kv.Kc && n0 >= kv.d) {
    const int which = n0 >= 2 * kv.d, c = n0 - (1 + which) * kv.d, h = c / kv.hs, e = c - h * kv.hs;
    st4((which ? kv.Vc : kv.Kc) + ((size_t)h * kv.ctx + kv.pos0 + r) * kv.hs + e, s);
  }
}

// gemv_reduce for the many slices of a matrix-vector product (S = K / 64): sixteen threads share an output
// float4, thread ty summing slices ty, ty + 16, ... (loads in flight together instead of S in a row), the
// sixteen sums combined in ascending ty by the first of them. Same result for every run; bias last.
__global__ __launch_bounds__(WG) void gemv_reduce_wide(int M, int N, int S, const float* __restrict__ part,
                                                        const float* __restrict__ bias, float* C, int ldc, int epi,
                                                        const float* resid) {
  __shared__ float4 red[16][16];
  const int n4 = N >> 2;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int idx = blockIdx.x * 16 + tx;
  const bool live = idx < M * n4;
  const int r = live ? idx / n4 : 0, n0 = live ? (idx - r * n4) * 4 : 0;
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  if (live) {
#pragma unroll 4
    for (int sp = ty; sp < S; sp += 16) {
      const float4 v = ld4(part + ((size_t)sp * M + r) * N + n0);
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
  }
  red[ty][tx] = s;
  __syncthreads();
  if (ty != 0 || !live) return;
#pragma unroll
  for (int j = 1; j < 16; ++j) {
    const float4 v = red[j][tx];
    s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
  }
  if (bias) {
    const float4 b = ld4(bias + n0);
    s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
  }
  if (epi == EPI_GELU) {
    s.x = gelu_ref(s.x); s.y = gelu_ref(s.y); s.z = gelu_ref(s.z); s.w = gelu_ref(s.w);
  } else if (epi == EPI_RESIDUAL) {
    const float4 q = ld4(resid + (size_t)r * ldc + n0);
    s.x += q.x; s.y += q.y; s.z += q.z; s.w += q.w;
  }
  st4(C + (size_t)r * ldc + n0, s);
}

// gemv_reduce of one row followed by the LayerNorm of that row (layernorm_kernel's arithmetic and order of
// operations, thread t holding the float4 t, t + WG, ... of the row): C gets the finished row, ln_out its
// normalisation. One workgroup per row; N a multiple of 4, at most 4 * WG * REDUCE_LN_MAXV.
constexpr int REDUCE_LN_MAXV = 4;
__global__ __launch_bounds__(WG) void reduce_ln_kernel(int M, int N, int S, const float* __restrict__ part,
                                                        const float* __restrict__ bias, float* C, int ldc, int epi,
                                                        const float* resid, const float* __restrict__ gamma,
                                                        const float* __restrict__ beta, float* __restrict__ ln_out, int ldo) {
  __shared__ float sh[NWAVE];
  const int r = blockIdx.x, n4 = N >> 2;
  float4 v[REDUCE_LN_MAXV], gpre[REDUCE_LN_MAXV], bpre[REDUCE_LN_MAXV];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < REDUCE_LN_MAXV; ++j) {
    const int i = threadIdx.x + j * WG;
    v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    gpre[j] = bpre[j] = v[j];
    if (i < n4) {
      const int n0 = 4 * i;
      // (requested with the partial sums: behind the two reductions they would be a memory round trip of their own)
      gpre[j] = ld4(gamma + n0);
      bpre[j] = ld4(beta + n0);
      float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int sp = 0; sp < S; ++sp) {
        const float4 p = ld4(part + ((size_t)sp * M + r) * N + n0);
        a.x += p.x; a.y += p.y; a.z += p.z; a.w += p.w;
      }
      if (bias) {
        const float4 b = ld4(bias + n0);
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
      }
      if (epi == EPI_GELU) {
        a.x = gelu_ref(a.x); a.y = gelu_ref(a.y); a.z = gelu_ref(a.z); a.w = gelu_ref(a.w);
      } else if (epi == EPI_RESIDUAL) {
        const float4 q = ld4(resid + (size_t)r * ldc + n0);
        a.x += q.x; a.y += q.y; a.z += q.z; a.w += q.w;
      }
      st4(C + (size_t)r * ldc + n0, a);
      v[j] = a;
      sum += (a.x + a.y) + (a.z + a.w);
    }
  }
  const float mean = block_sum(sum, sh) / (float)N;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < REDUCE_LN_MAXV; ++j) {
    if (threadIdx.x + j * WG < n4) {
      const float a = v[j].x - mean, b = v[j].y - mean, c = v[j].z - mean, d = v[j].w - mean;
      q += (a * a + b * b) + (c * c + d * d);
    }
  }
  const float var = block_sum(q, sh) / (float)N;
  const float stdev = sqrtf(var + 1e-5f);
#pragma unroll
  for (int j = 0; j < REDUCE_LN_MAXV; ++j) {
    const int i = threadIdx.x + j * WG;
    if (i < n4) {
      const float4 g = gpre[j], b = bpre[j];
      float4 o;
      o.x = g.x * ((v[j].x - mean) / stdev) + b.x;
      o.y = g.y * ((v[j].y - mean) / stdev) + b.y;
      o.z = g.z * ((v[j].z - mean) / stdev) + b.z;
      o.w = g.w * ((v[j].w - mean) / stdev) + b.w;
      st4(ln_out + (size_t)r * ldo + 4 * i, o);
    }
  }
}

// int8 weight-only stage 1 (other/int8-gemm.js:156-210 at M <= 4): a wave reads
// 64 consecutive words (256 columns) of one row; 4 waves take rows k0+ty, +4, ...
template <int R>
__global__ __launch_bounds__(WG) void gemv_kn_i8_partial(int N, int K, const float* __restrict__ A, int lda,
                                                          const int32_t* __restrict__ Wq, int ldwq,
                                                          const float* __restrict__ scale, float* __restrict__ part) {
  __shared__ float4 red[R][NWAVE][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 256 + tx * 4;
  const int k0 = blockIdx.y * GEMV_KCHUNK;
  float4 acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
  if (n0 < N) {
    const float4 sc = ld4(scale + n0);
#pragma unroll 4
    for (int i = 0; i < GEMV_KCHUNK / NWAVE; ++i) {
      const int k = k0 + ty + NWAVE * i;
      if (k < K) {
        const float4 w = unpack_i8x4(Wq[(size_t)k * ldwq + (n0 >> 2)], sc);
#pragma unroll
        for (int r = 0; r < R; ++r) fma4(acc[r], A[(size_t)r * lda + k], w);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) red[r][ty][tx] = acc[r];
  __syncthreads();
  if (ty < R && n0 < N) {
    float4 s = red[ty][0][tx];
#pragma unroll
    for (int j = 1; j < NWAVE; ++j) {
      const float4 v = red[ty][j][tx];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    st4(part + ((size_t)blockIdx.y * R + ty) * N + n0, s);
  }
}

__global__ __launch_bounds__(WG) void dequant_i8_kernel(int K, int N, const int32_t* __restrict__ Wq, int ldwq,
                                                         const float* __restrict__ scale, float* __restrict__ W, int ldw) {
  const int n4 = N >> 2;
  const size_t idx = (size_t)blockIdx.x * WG + threadIdx.x;
  if (idx >= (size_t)K * n4) return;
  const int k = (int)(idx / n4), w = (int)(idx - (size_t)k * n4);
  st4(W + (size_t)k * ldw + 4 * w, unpack_i8x4(Wq[(size_t)k * ldwq + w], ld4(scale + 4 * w)));
}

// ---------------------------------------------------------------------------
// FastMatMulBlock for any M (prefill): 64x64 output tile per workgroup, 4x4 per
// thread, K in steps of 16 through LDS. Same contraction and bias-last order of
// operations per element as instructions.js:248-314 up to fp32 reassociation.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(WG) void gemm_tile64(int M, int N, int K, const float* __restrict__ A, int lda,
                                                   const float* __restrict__ W, int ldw, const float* __restrict__ bias,
                                                   float* C, int ldc, int epi, const float* resid) {
  __shared__ float As[16][64 + 4];
  __shared__ float Bs[16][64];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tm = tid >> 4, tn = tid & 15;
  const int arow = tid >> 2, akq = (tid & 3) * 4;
  const int brow = tid >> 4, bnq = (tid & 15) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += 16) {
    float4 av = make_float4(0.f, 0.f, 0.f, 0.f), bv = make_float4(0.f, 0.f, 0.f, 0.f);
    if (m0 + arow < M && k0 + akq < K) av = ld4(A + (size_t)(m0 + arow) * lda + k0 + akq);
    if (k0 + brow < K && n0 + bnq < N) bv = ld4(W + (size_t)(k0 + brow) * ldw + n0 + bnq);
    As[akq + 0][arow] = av.x;
    As[akq + 1][arow] = av.y;
    As[akq + 2][arow] = av.z;
    As[akq + 3][arow] = av.w;
    st4(&Bs[brow][bnq], bv);
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      const float4 a = ld4(&As[kk][tm * 4]);
      const float4 b = ld4(&Bs[kk][tn * 4]);
      const float aa[4] = {a.x, a.y, a.z, a.w};
      const float bb[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += aa[i] * bb[j];
    }
    __syncthreads();
  }
  const int n = n0 + tn * 4;
  if (n >= N) return;
  float4 b = make_float4(0.f, 0.f, 0.f, 0.f);
  if (bias) b = ld4(bias + n);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tm * 4 + i;
    if (m >= M) break;
    float4 v = make_float4(acc[i][0] + b.x, acc[i][1] + b.y, acc[i][2] + b.z, acc[i][3] + b.w);
    if (epi == EPI_GELU) {
      v.x = gelu_ref(v.x); v.y = gelu_ref(v.y); v.z = gelu_ref(v.z); v.w = gelu_ref(v.w);
    } else if (epi == EPI_RESIDUAL) {
      const float4 q = ld4(resid + (size_t)m * ldc + n);
      v.x += q.x; v.y += q.y; v.z += q.z; v.w += q.w;
    }
    st4(C + (size_t)m * ldc + n, v);
  }
}


// ---------------------------------------------------------------------------
// FastMatMulBlock as a dense contraction on the matrix cores (prefill, M >= 16):
// C = epi(A . W + bias). fp32 MFMA v_mfma_f32_32x32x2_f32: per instruction a wave
// multiplies a 32x2 slice of A by a 2x32 slice of W into a 32x32 fp32 accumulator
// (16 VGPRs per lane). Workgroup tile TM x TN (64 or 128 each), four waves in a 2x2
// arrangement, each owning (TM/2) x (TN/2) of C as RB x CB accumulator blocks, so an
// operand fragment read from LDS feeds CB (or RB) instructions. K advances in steps
// of BK = 32 through two LDS stages (one barrier per step); inside a step every wave
// interleaves its matrix instructions with the LDS reads of the next quarter-step, the
// global loads of a later step and the move of the next step into the other stage.
// A is staged as [m][BK + 4] with the k of a step permuted to (k odd, k / 2), so the
// values a lane feeds to four consecutive instructions are one 128-bit read; W as
// [k][n], odd k with the two 32-column halves of a row swapped so that the two half-waves
// of an operand read (k and k + 1) use different LDS banks.
// Operand lane mapping of the instruction: lane l supplies A[row l%32][k l/32] and
// W[k l/32][col l%32]; accumulator register r of lane l is
// C[row (r/4)*8 + (l/32)*4 + r%4][col l%32].
// ---------------------------------------------------------------------------
typedef float f32x16 __attribute__((ext_vector_type(16)));

// With kchunk < K (split-K) slice blockIdx.z covers k in [z*kchunk, (z+1)*kchunk) and
// writes its raw partial sums to C + z*M*ldc (bias, epilogue: gemv_reduce afterwards).
// I8W: W is the packed int8 matrix of other/int8-gemm.js:36-43 (`Wv` points to [K, ldw] words of four
// consecutive columns, `wscale` to the per-column scales); a thread's word of a step is
// dequantised on its way into LDS with the arithmetic of unpackInt8x4, so the matrix cores
// see exactly the weights wgpt_dequant_i8 would write, without the trip through memory.
template <int TM, int TN, int BK, bool I8W, bool EXACT>
__global__ __launch_bounds__(WG) void gemm_mfma(int M, int N, int K, int kchunk, const float* __restrict__ A, int lda,
                                                 const void* __restrict__ Wv, int ldw, const float* __restrict__ wscale,
                                                 const float* __restrict__ bias, float* C, int ldc, int epi, const float* resid) {
  const float* W = static_cast<const float*>(Wv);
  const int32_t* Wq = static_cast<const int32_t*>(Wv);
  constexpr int AST = BK + 4;                // floats per staged A row (16-byte aligned, odd multiple of 4 banks)
  constexpr int RB = TM / 64, CB = TN / 64;  // 32x32 accumulator blocks per wave
  constexpr int KQ = BK / 4;                 // float4 per A row of a step
  constexpr int AROWS = WG / KQ;             // A rows covered by one pass of the workgroup
  constexpr int NA = TM / AROWS;             // float4 per thread of the A tile of a step
  constexpr int BROWS = WG / (TN / 4);       // W rows covered by one pass of the workgroup
  constexpr int NB = BK / BROWS;             // float4 per thread of the W tile of a step
  constexpr int HK = BK / 2;                 // MFMA instructions per step and accumulator block
  constexpr int NQ = HK / 4;                 // quarters of a step: four k pairs each
  constexpr int BST = TN;                    // floats per staged W row (odd rows swap their 32-column halves)
  __shared__ __attribute__((aligned(16))) float As[2][TM * AST];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * BST];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int wm = (wave >> 1) * (TM / 2), wn = (wave & 1) * (TN / 2);
  const int arow = tid / KQ, akq = (tid % KQ) * 4;
  const int brow = tid / (TN / 4), bnq = (tid % (TN / 4)) * 4;
  // D register sets of global data: a step's tile is fetched D steps ahead of its use and moves into
  // LDS one step ahead; with two sets, set p holds the steps of parity p
  constexpr int D = RB * CB == 1 ? 2 : 1;  // the large tile has registers for one set only
  float4 ga[D][NA], gb[D][I8W ? 1 : NB];
  int32_t gq[D][I8W ? NB : 1];  // packed words of the step, unpacked when they are staged
  float4 sc4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (I8W && n0 + bnq < N) sc4 = ld4(wscale + n0 + bnq);
  // Every global load is unconditional and in bounds: rows beyond M and columns beyond N repeat the
  // last valid ones (their results are never stored), k beyond the slice repeats its last values and is
  // zeroed when the step is staged. (A load under a bounds branch makes the compiler wait for it on
  // the spot, which exposes the whole memory latency in every step.) EXACT: every K slice is whole
  // steps, so there is nothing to clamp or zero along k, and a step's addresses are a uniform base
  // plus per-thread offsets: vector-ALU instructions of a step queue behind the matrix instructions
  // of the other waves of the SIMD, so the fewer the better.
  const int kbeg = blockIdx.z * kchunk;
  const int kend = kbeg + kchunk < K ? kbeg + kchunk : K;
  C += (size_t)blockIdx.z * M * ldc;
  K = kend;
  const int ncl = n0 + bnq < N ? n0 + bnq : N - 4;
  unsigned aoff[NA], boff[NB];  // element offsets from the step's first k (A) / first row (W)
#pragma unroll
  for (int r = 0; r < NA; ++r) {
    const int m = m0 + arow + r * AROWS;
    aoff[r] = (unsigned)((size_t)(m < M ? m : M - 1) * lda + akq);
  }
#pragma unroll
  for (int r = 0; r < NB; ++r) boff[r] = (unsigned)((size_t)(brow + r * BROWS) * ldw + (I8W ? ncl >> 2 : ncl));
  int kf[D] = {};  // first k of the step held by each set
  auto fetch = [&](auto P, int k0) {
    constexpr int p = decltype(P)::value;
    kf[p] = k0;
    if (EXACT) {
      const float* at = A + k0;
      const size_t wrow = (size_t)k0 * ldw;
#pragma unroll
      for (int r = 0; r < NA; ++r) ga[p][r] = ld4(at + aoff[r]);
#pragma unroll
      for (int r = 0; r < NB; ++r) {
        if (I8W) gq[p][I8W ? r : 0] = (Wq + wrow)[boff[r]];
        else gb[p][I8W ? 0 : r] = ld4(W + wrow + boff[r]);
      }
    } else {
      const int ka = k0 + akq < K ? k0 : K - 4 - akq;
#pragma unroll
      for (int r = 0; r < NA; ++r) ga[p][r] = ld4(A + ka + aoff[r]);
#pragma unroll
      for (int r = 0; r < NB; ++r) {
        const int k = k0 + brow + r * BROWS;
        const size_t wrow = (size_t)(k < K ? k0 : K - 1 - brow - r * BROWS) * ldw;
        if (I8W) gq[p][I8W ? r : 0] = (Wq + wrow)[boff[r]];
        else gb[p][I8W ? 0 : r] = ld4(W + wrow + boff[r]);
      }
    }
  };
  // LDS layouts: A tile as [m][BK + 4], W tile as [k][TN] with the two 32-column halves of every 64 columns
  // swapped in rows with bit 2 set. Matrix instruction i of quarter q takes k = 8q + 4h + i from half-wave h, so
  // a lane's four A values of a quarter are one 128-bit read of the unpermuted row, and the two half-waves of
  // a W read (rows 8q + i and 8q + 4 + i) use different banks.
  auto stage = [&](auto P, int st) {
    constexpr int p = decltype(P)::value;
    const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    const bool ain = EXACT || kf[p] + akq < K;
#pragma unroll
    for (int r = 0; r < NA; ++r) st4(As[st] + (arow + r * AROWS) * AST + akq, ain ? ga[p][r] : z);
#pragma unroll
    for (int r = 0; r < NB; ++r) {
      const int row = brow + r * BROWS;
      const bool bin = EXACT || kf[p] + row < K;
      const float4 v = I8W ? unpack_i8x4(gq[p][I8W ? r : 0], sc4) : gb[p][I8W ? 0 : r];
      st4(Bs[st] + row * BST + (bnq ^ (((row >> 2) & 1) << 5)), bin ? v : z);
    }
  };
  f32x16 acc[RB][CB];
#pragma unroll
  for (int r = 0; r < RB; ++r)
#pragma unroll
    for (int c = 0; c < CB; ++c)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[r][c][i] = 0.f;

  const int h = lane >> 5, l32 = lane & 31;
  // operands of quarter q of the step in LDS stage st: four k pairs per accumulator row / column block
  auto operands = [&](float (&av)[RB][4], float (&bv)[CB][4], int st, int q) {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const float4 v = ld4(As[st] + (wm + r * 32 + l32) * AST + 8 * q + 4 * h);
      av[r][0] = v.x; av[r][1] = v.y; av[r][2] = v.z; av[r][3] = v.w;
    }
#pragma unroll
    for (int c = 0; c < CB; ++c) {
      const float* bp = Bs[st] + (8 * q + 4 * h) * BST + ((wn + c * 32 + l32) ^ (h << 5));
#pragma unroll
      for (int i = 0; i < 4; ++i) bv[c][i] = bp[i * BST];
    }
  };
  auto multiply = [&](const float (&av)[RB][4], const float (&bv)[CB][4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int c = 0; c < CB; ++c) acc[r][c] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[r][i], bv[c][i], acc[r][c], 0, 0, 0);
  };

  // requested before the main loop so that the epilogue does not wait for it
  float biasv[CB];
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    const int n = n0 + wn + c * 32 + l32;
    biasv[c] = (bias && n < N) ? bias[n] : 0.f;
  }
  typedef std::integral_constant<int, 0> P0;
  typedef std::integral_constant<int, 1> P1;
  fetch(P0(), kbeg);
  stage(P0(), 0);
  if constexpr (D == 2) {
    if (kbeg + BK < kend) fetch(P1(), kbeg + BK);
  }
  __syncthreads();
  float av[2][RB][4], bv[2][CB][4];  // operands of the quarter being multiplied and of the next one
  operands(av[0], bv[0], 0, 0);
  int st = 0;
  // One K step. A wave keeps its own matrix pipe fed: while the instructions of a quarter run, the
  // operands of the next quarter are on their way from LDS, the global loads of a later step (D steps
  // ahead) are in flight, and the next step's tile moves from registers into the other LDS stage. The
  // last quarter is multiplied after the barrier, behind the request for the next step's first
  // operands. (Leaving the overlap to a second wave of the SIMD does not work: the workgroups of a
  // compute unit fall into step with each other and stall together.)
  // FETCH / STAGE are compile-time so that the steady state is straight-line code: with a branch
  // around the loads the compiler can no longer tell which of them are outstanding and waits early.
  auto kstep = [&](auto P, auto FETCH, auto STAGE, int k0) {
    constexpr int p = decltype(P)::value;
    static_assert(NQ % 2 == 0, "the last quarter of a step must sit in operand set 1");
    if (decltype(FETCH)::value) {
      fetch(std::integral_constant<int, D == 2 ? p : 0>(), k0 + D * BK);  // that set was staged a step ago
      __builtin_amdgcn_sched_barrier(0);  // keep the loads here, at the head of the step
    }
#pragma unroll
    for (int q = 0; q < NQ - 1; ++q) {
      operands(av[(q + 1) & 1], bv[(q + 1) & 1], st, q + 1);
      multiply(av[q & 1], bv[q & 1]);
    }
    if (decltype(STAGE)::value) {
      __builtin_amdgcn_sched_barrier(0);  // nothing of the move into LDS (it waits for the loads) drifts up
      stage(std::integral_constant<int, D == 2 ? 1 - p : 0>(), st ^ 1);
      __syncthreads();
      st ^= 1;
      operands(av[0], bv[0], st, 0);
    }
    multiply(av[1], bv[1]);
  };
  const std::true_type yes;
  const std::false_type no;
  int k0 = kbeg;
  if constexpr (D == 2) {
    for (; k0 + 3 * BK < kend; k0 += 2 * BK) {
      kstep(P0(), yes, yes, k0);
      kstep(P1(), yes, yes, k0 + BK);
    }
    if (k0 + 2 * BK < kend) {  // three steps left
      kstep(P0(), yes, yes, k0);
      kstep(P1(), no, yes, k0 + BK);
      kstep(P0(), no, no, k0 + 2 * BK);
    } else if (k0 + BK < kend) {  // two
      kstep(P0(), no, yes, k0);
      kstep(P1(), no, no, k0 + BK);
    } else if (k0 < kend) {  // one
      kstep(P0(), no, no, k0);
    }
  } else {
    for (; k0 + BK < kend; k0 += BK) kstep(P0(), yes, yes, k0);
    if (k0 < kend) kstep(P0(), no, no, k0);
  }
#pragma unroll
  for (int c = 0; c < CB; ++c) {
    const int n = n0 + wn + c * 32 + l32;
    if (n >= N) continue;
    const float bvs = biasv[c];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int m = m0 + wm + r * 32 + (i >> 2) * 8 + h * 4 + (i & 3);
        if (m < M) {
          float v = acc[r][c][i] + bvs;
          if (epi == EPI_GELU) v = gelu_ref(v);
          else if (epi == EPI_RESIDUAL) v += resid[(size_t)m * ldc + n];
          C[(size_t)m * ldc + n] = v;
        }
      }
  }
}

// ---------------------------------------------------------------------------
// The same contraction for problems that give every compute unit one 64 x 128 tile: 512 threads, two
// groups of four waves (one wave of each group per SIMD); group g owns columns [64g, 64g + 64) of the
// tile, its waves a 32 x 32 block each. The groups alternate: while one issues the 16 matrix
// instructions of a K step from registers, the other does its memory work (operands of its next
// step from LDS into registers, its share of a later tile from registers into LDS, global loads two
// steps ahead of that), then they swap at a barrier. A SIMD's matrix pipe therefore always has
// exactly one wave feeding it, and no wave waits for memory between matrix instructions. (With
// independent workgroups the waves of a SIMD run in step, want the pipe at the same time and stall
// at the same time.) Tiles of K steps 0, 1, ... alternate between two LDS stages; group 0 multiplies
// step k in the first half of iteration k, group 1 in the second half. Every load and LDS write is
// unconditional: tiles beyond the K range are fetched from clamped addresses and staged as zeros.
// ---------------------------------------------------------------------------
constexpr int PP_THREADS = 512;
constexpr int PP_BK = 32;  // K step (64 measured 3-5 % slower)
constexpr size_t PP_LDS = sizeof(float) * 2 * (64 * (PP_BK + 4) + PP_BK * 128);
template <int BK>
__global__ __launch_bounds__(PP_THREADS) void gemm_pingpong(int M, int N, int K, int kchunk, const float* __restrict__ A, int lda,
                                                            const float* __restrict__ W, int ldw, const float* __restrict__ bias,
                                                            float* C, int ldc, int epi, const float* resid) {
  constexpr int TM = 64, TN = 128, AST = BK + 4, HK = BK / 2;
  constexpr int NA = BK / 32, NB = BK / 16;  // float4 of A and of W per thread and tile
  extern __shared__ __attribute__((aligned(16))) float pp_lds[];
  float* const As = pp_lds;                  // [2][TM * AST]
  float* const Bs = pp_lds + 2 * TM * AST;   // [2][BK * TN]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = wave >> 2, wq = wave & 3, t = tid & 255;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int wm = (wq >> 1) * 32, wn = g * 64 + (wq & 1) * 32;
  const int h = lane >> 5, l32 = lane & 31;
  // this thread's share of a tile: NA float4 of A (row 32g + t / 8, float4 t % 8 + 8j of the row), NB of W (the
  // group's own columns, rows t / 16 + 16r). Rows beyond M and columns beyond N repeat the last valid ones
  // (their results are never stored).
  const int arow = g * 32 + (t >> 3), akq = (t & 7) * 4;
  const int brow = t >> 4, bnq = g * 64 + (t & 15) * 4;
  const int ncl = n0 + bnq < N ? n0 + bnq : N - 4;
  // byte offsets of the thread inside a tile; the tile's own address is uniform and advances with the step,
  // so that a memory phase issues almost no vector-ALU instructions: those queue behind the other group's
  // matrix instructions on the same SIMD, LDS and global-memory instructions do not
  unsigned aoff[NA], boff[NB];
#pragma unroll
  for (int j = 0; j < NA; ++j) aoff[j] = (unsigned)(((size_t)(m0 + arow < M ? m0 + arow : M - 1) * lda + akq + 32 * j) * sizeof(float));
#pragma unroll
  for (int j = 0; j < NB; ++j) boff[j] = (unsigned)(((size_t)(brow + 16 * j) * ldw + ncl) * sizeof(float));

  const int kbeg = blockIdx.z * kchunk;
  const int kend = kbeg + kchunk < K ? kbeg + kchunk : K;
  C += (size_t)blockIdx.z * M * ldc;
  const int nsteps = (kend - kbeg) / BK;  // the launcher guarantees whole steps
  const char* Abase = reinterpret_cast<const char*>(A + kbeg);
  const char* Wbase = reinterpret_cast<const char*>(W + (size_t)kbeg * ldw);
  const size_t wstep = (size_t)BK * ldw * sizeof(float);

  struct Share {
    float4 a[NA], b[NB];
  };
  auto load_share = [&](int tile) {  // this thread's share of tile `tile` (tiles past the end repeat the last one)
    const int tc = tile < nsteps ? tile : nsteps - 1;
    // the tile addresses are uniform: keep them in scalar registers
    const unsigned long long wo = (unsigned long long)tc * wstep;
    const unsigned wlo = __builtin_amdgcn_readfirstlane((unsigned)wo), whi = __builtin_amdgcn_readfirstlane((unsigned)(wo >> 32));
    const char* at = Abase + __builtin_amdgcn_readfirstlane(tc * (int)(BK * sizeof(float)));
    const char* wt = Wbase + (((unsigned long long)whi << 32) | wlo);
    Share r;
#pragma unroll
    for (int j = 0; j < NA; ++j) r.a[j] = *reinterpret_cast<const float4*>(at + aoff[j]);
#pragma unroll
    for (int j = 0; j < NB; ++j) r.b[j] = *reinterpret_cast<const float4*>(wt + boff[j]);
    return r;
  };
  Share set[2];
  auto fetch = [&](auto P, int tile) { set[decltype(P)::value] = load_share(tile); };
  // LDS layouts: A tile as [m][BK + 4], W tile as [k][TN] with the two 32-column halves of a 64-column group
  // swapped in rows with bit 2 set. Matrix instruction i of quarter q takes k = 8q + 4h + i from half-wave h, so a
  // lane's four A values of a quarter are one 128-bit read of the unpermuted row, and the two half-waves of a W
  // read (rows 8q + i and 8q + 4 + i) use different banks.
  float* const adst = As + arow * AST + akq;
  float* const bdst = Bs + brow * TN + (bnq ^ (((brow >> 2) & 1) << 5));  // rows + 16r have the same bit 2
  auto stage = [&](auto P, int st) {  // set p -> LDS stage st
    constexpr int p = decltype(P)::value;
#pragma unroll
    for (int j = 0; j < NA; ++j) st4(adst + st * (TM * AST) + 32 * j, set[p].a[j]);
#pragma unroll
    for (int j = 0; j < NB; ++j) st4(bdst + st * (BK * TN) + 16 * j * TN, set[p].b[j]);
  };
  float av[HK], bv[HK];
  const float* const asrc = As + (wm + l32) * AST + 4 * h;
  const float* const bsrc = Bs + 4 * h * TN + ((wn + l32) ^ (h << 5));
  auto operands = [&](int st) {  // the wave's operands of a whole K step
#pragma unroll
    for (int q = 0; q < HK / 4; ++q) {
      const float4 v = ld4(asrc + st * (TM * AST) + 8 * q);
      av[4 * q] = v.x; av[4 * q + 1] = v.y; av[4 * q + 2] = v.z; av[4 * q + 3] = v.w;
#pragma unroll
      for (int i = 0; i < 4; ++i) bv[4 * q + i] = bsrc[st * (BK * TN) + (8 * q + i) * TN];
    }
  };
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  auto multiply = [&]() {
#pragma unroll
    for (int i = 0; i < HK; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[i], acc, 0, 0, 0);
  };
  const int n = n0 + wn + l32;
  const float bvs = (bias && n < N) ? bias[n] : 0.f;  // requested early: the epilogue does not wait for it

  typedef std::integral_constant<int, 0> P0;
  typedef std::integral_constant<int, 1> P1;
  // the matrix instructions touch registers only, so the scheduler would move them across a barrier into the
  // memory phase and undo the alternation: pin both sides
  auto phase_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };
  // Tile j lives in LDS stage j & 1 and travels through register set j & 1. The two groups run separate
  // loops with the same number of barriers (1 + 2 * nsteps), so that no value has to be merged between
  // their code paths.
  if (g == 0) {
    // multiplies step k in the first half of iteration k; leads by two tiles: 0 and 1 staged, 2 and 3 in flight
    fetch(P0(), 0);
    fetch(P1(), 1);
    const Share t2 = load_share(2), t3 = load_share(3);  // requested before the first two are waited for
    stage(P0(), 0);
    stage(P1(), 1);
    set[0] = t2;
    set[1] = t3;
    phase_barrier();
    operands(0);
    auto iteration = [&](auto parity, int k) {
      typedef decltype(parity) P;
      multiply();  // step k
      phase_barrier();
      operands(1 - P::value);  // step k + 1
      stage(P(), P::value);    // tile k + 2
      fetch(P(), k + 4);
      phase_barrier();
    };
    int k = 0;
    for (; k + 1 < nsteps; k += 2) {
      iteration(P0(), k);
      iteration(P1(), k + 1);
    }
    if (k < nsteps) iteration(P0(), k);
  } else {
    // multiplies step k in the second half of iteration k; leads by one tile: 0 staged, 1 and 2 in flight
    fetch(P0(), 0);
    fetch(P1(), 1);
    const Share t2 = load_share(2);
    stage(P0(), 0);
    set[0] = t2;
    phase_barrier();
    auto iteration = [&](auto parity, int k) {
      typedef decltype(parity) P;
      typedef std::integral_constant<int, 1 - P::value> Q;
      operands(P::value);      // step k
      stage(Q(), Q::value);    // tile k + 1
      fetch(Q(), k + 3);
      phase_barrier();
      multiply();  // step k
      phase_barrier();
    };
    int k = 0;
    for (; k + 1 < nsteps; k += 2) {
      iteration(P0(), k);
      iteration(P1(), k + 1);
    }
    if (k < nsteps) iteration(P0(), k);
  }

  if (n < N) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = m0 + wm + (i >> 2) * 8 + h * 4 + (i & 3);
      if (m < M) {
        float v = acc[i] + bvs;
        if (epi == EPI_GELU) v = gelu_ref(v);
        else if (epi == EPI_RESIDUAL) v += resid[(size_t)m * ldc + n];
        C[(size_t)m * ldc + n] = v;
      }
    }
  }
}

// ResidualBlock, instructions.js:381-382
__global__ __launch_bounds__(WG) void residual_kernel(size_t n4, const float* a, const float* b, float* out) {
  const size_t i = (size_t)blockIdx.x * WG + threadIdx.x;
  if (i >= n4) return;
  const float4 x = ld4(a + 4 * i), y = ld4(b + 4 * i);
  st4(out + 4 * i, make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w));
}

// GeluBlock, instructions.js:718-746
__global__ __launch_bounds__(WG) void gelu_kernel(size_t n4, const float* x, float* out) {
  const size_t i = (size_t)blockIdx.x * WG + threadIdx.x;
  if (i >= n4) return;
  const float4 v = ld4(x + 4 * i);
  st4(out + 4 * i, make_float4(gelu_ref(v.x), gelu_ref(v.y), gelu_ref(v.z), gelu_ref(v.w)));
}

// LayerNormBlock: stats pass + norm pass of instructions.js:451-550 in one kernel,
// one workgroup per row. mean = sum/N; var = sum((x-mean)^2)/N; stdev = sqrt(var + 1e-5);
// out = gamma * ((x - mean) / stdev) + beta with a true division.
__global__ __launch_bounds__(WG) void layernorm_kernel(int N, const float* __restrict__ x, int ldx,
                                                        const float* __restrict__ gamma, const float* __restrict__ beta,
                                                        float* __restrict__ out, int ldo) {
  __shared__ float sh[NWAVE];
  const float* xr = x + (size_t)blockIdx.x * ldx;
  float* orow = out + (size_t)blockIdx.x * ldo;
  const int n4 = N >> 2;
  float s = 0.f;
  for (int i = threadIdx.x; i < n4; i += WG) {
    const float4 v = ld4(xr + 4 * i);
    s += (v.x + v.y) + (v.z + v.w);
  }
  const float mean = block_sum(s, sh) / (float)N;
  float q = 0.f;
  for (int i = threadIdx.x; i < n4; i += WG) {
    const float4 v = ld4(xr + 4 * i);
    const float a = v.x - mean, b = v.y - mean, c = v.z - mean, d = v.w - mean;
    q += (a * a + b * b) + (c * c + d * d);
  }
  const float var = block_sum(q, sh) / (float)N;
  const float stdev = sqrtf(var + 1e-5f);
  for (int i = threadIdx.x; i < n4; i += WG) {
    const float4 v = ld4(xr + 4 * i), g = ld4(gamma + 4 * i), b = ld4(beta + 4 * i);
    float4 o;
    o.x = g.x * ((v.x - mean) / stdev) + b.x;
    o.y = g.y * ((v.y - mean) / stdev) + b.y;
    o.z = g.z * ((v.z - mean) / stdev) + b.z;
    o.w = g.w * ((v.w - mean) / stdev) + b.w;
    st4(orow + 4 * i, o);
  }
}

// SoftmaxBlock, instructions.js:618-663: max from -3.402823e38, sum of exp(x - max),
// out = exp(x - max) / sum with the exponential recomputed and a true division.
// TRANSPOSE: the store of instructions.js:594 with `transpose` set: element i of row r goes to out[i * M + r].
template <bool TRANSPOSE>
__global__ __launch_bounds__(WG) void softmax_kernel(int M, int N, const float* __restrict__ x, float* __restrict__ out) {
  __shared__ float sh[NWAVE];
  const float* xr = x + (size_t)blockIdx.x * N;
  float* orow = out + (size_t)blockIdx.x * N;
  float m = -3.402823e+38f;
  for (int i = threadIdx.x; i < N; i += WG) m = fmaxf(m, xr[i]);
  m = block_max(m, sh);
  float s = 0.f;
  for (int i = threadIdx.x; i < N; i += WG) s += expf(xr[i] - m);
  s = block_sum(s, sh);
  for (int i = threadIdx.x; i < N; i += WG) {
    const float v = expf(xr[i] - m) / s;
    if (TRANSPOSE) out[(size_t)i * M + blockIdx.x] = v;
    else orow[i] = v;
  }
}

// out[c * rows + r] = in[r * cols + c] through a 32 x 32 tile of LDS (the host-side transpose of globals.js:80-94).
__global__ __launch_bounds__(256) void transpose_kernel(int rows, int cols, const float* __restrict__ in, float* __restrict__ out) {
  __shared__ float tile[32][33];
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
  const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
  for (int k = ty; k < 32; k += 8)
    if (r0 + k < rows && c0 + tx < cols) tile[k][tx] = in[(size_t)(r0 + k) * cols + c0 + tx];
  __syncthreads();
  for (int k = ty; k < 32; k += 8)
    if (c0 + k < cols && r0 + tx < rows) out[(size_t)(c0 + k) * rows + r0 + tx] = tile[tx][k];
}

// EmbedBlock, instructions.js:795-821: gather + positional add in one pass.
__global__ __launch_bounds__(WG) void embed_kernel(const int32_t* __restrict__ idx, int d, int pos0,
                                                    const float* __restrict__ wte, const float* __restrict__ wpe,
                                                    float* __restrict__ out, const int* __restrict__ pos_dev = nullptr) {
  const int i = blockIdx.x;
  if (pos_dev) pos0 = *pos_dev;
  const size_t tok = (size_t)idx[i];
  const float* e = wte + tok * d;
  const float* p = wpe + (size_t)(pos0 + i) * d;
  for (int c = threadIdx.x; c < (d >> 2); c += WG) {
    const float4 a = ld4(e + 4 * c), b = ld4(p + 4 * c);
    st4(out + (size_t)i * d + 4 * c, make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w));
  }
}

// DeEmbedBlock, instructions.js:916-943, on the un-chunked, un-transposed wte[V,d]:
// row-major wte already has the contraction index contiguous, so a wave streams
// whole rows with 128-bit loads and reduces by shuffles. 4 rows per wave in flight.
constexpr int VOCAB_ROWS_PER_WAVE = 4;
__global__ __launch_bounds__(WG) void vocab_gemv_kernel(int V, int d, const float* __restrict__ x,
                                                         const float* __restrict__ wte, float* __restrict__ logits) {
  extern __shared__ __attribute__((aligned(16))) float xs[];
  for (int c = threadIdx.x; c < (d >> 2); c += WG) st4(xs + 4 * c, ld4(x + 4 * c));
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int v0 = (blockIdx.x * NWAVE + wave) * VOCAB_ROWS_PER_WAVE;
  float acc[VOCAB_ROWS_PER_WAVE];
#pragma unroll
  for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) acc[r] = 0.f;
  for (int c = lane; c < (d >> 2); c += 64) {
    const float4 xv = ld4(xs + 4 * c);
#pragma unroll
    for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) {
      if (v0 + r < V) {
        const float4 w = ld4(wte + (size_t)(v0 + r) * d + 4 * c);
        acc[r] += (xv.x * w.x + xv.y * w.y) + (xv.z * w.z + xv.w * w.w);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) {
    const float s = wave_sum(acc[r]);
    if (lane == 0 && v0 + r < V) logits[v0 + r] = s;
  }
}

// AttentionBlock's formatQ + fusedWeights + softmax + attentionValues
// (instructions.js:1129-1136, 1167-1176, 618-663, 1205-1212) for one (head, query
// row) per workgroup, reading K and V rows 0..p of head h at Kc + h*hstride + j*ldkv. Masked
// positions j > p get weight exactly 0 in the reference (exp(-1e9 - max) underflows),
// so they are skipped rather than multiplied by zero.
__global__ __launch_bounds__(WG) void attention_kernel(int pos0, int hs, int lpk, float scale, const float* __restrict__ q,
                                                        int ldq, const float* __restrict__ Kc, const float* __restrict__ Vc,
                                                        size_t hstride, int ldkv, float* __restrict__ out, int ldo) {
  extern __shared__ __attribute__((aligned(16))) float scores[];
  __shared__ __attribute__((aligned(16))) float qs[256];  // read as float4
  __shared__ float red[1024];
  __shared__ float sh[NWAVE];
  const int h = blockIdx.x, i = blockIdx.y;
  const int nkeys = pos0 + i + 1;
  const int tid = threadIdx.x;
  if (tid < hs) qs[tid] = q[(size_t)i * ldq + h * hs + tid];
  __syncthreads();
  const int sub = tid & (lpk - 1), grp = tid / lpk, ngrp = WG / lpk;
  const bool act = sub * 4 < hs;
  const float4 qv = act ? ld4(qs + sub * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
  const float* kbase = Kc + h * hstride + sub * 4;
  const float* vbase = Vc + h * hstride + sub * 4;
  // eight key rows per lane group requested before the first is used: one after the other, the ~24 rounds of a
  // 380-key context each waited a full memory round trip
  for (int j0 = 0; j0 < nkeys; j0 += 8 * ngrp) {
    float4 kv[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int j = j0 + u * ngrp + grp;
      kv[u] = (act && j < nkeys) ? ld4(kbase + (size_t)j * ldkv) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int j = j0 + u * ngrp + grp;
      float part = (qv.x * kv[u].x + qv.y * kv[u].y) + (qv.z * kv[u].z + qv.w * kv[u].w);
      for (int off = lpk >> 1; off > 0; off >>= 1) part += __shfl_xor(part, off);
      if (sub == 0 && j < nkeys) scores[j] = part * scale;
    }
  }
  __syncthreads();
  float m = -3.402823e+38f;
  for (int j = tid; j < nkeys; j += WG) m = fmaxf(m, scores[j]);
  m = block_max(m, sh);
  float s = 0.f;
  for (int j = tid; j < nkeys; j += WG) {
    const float e = expf(scores[j] - m);
    scores[j] = e;
    s += e;
  }
  s = block_sum(s, sh);
  for (int j = tid; j < nkeys; j += WG) scores[j] = scores[j] / s;
  __syncthreads();
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (act) {
    int j = grp;
    for (; j + 7 * ngrp < nkeys; j += 8 * ngrp) {
      float4 vv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) vv[u] = ld4(vbase + (size_t)(j + u * ngrp) * ldkv);
#pragma unroll
      for (int u = 0; u < 8; ++u) fma4(acc, scores[j + u * ngrp], vv[u]);
    }
    for (; j < nkeys; j += ngrp) fma4(acc, scores[j], ld4(vbase + (size_t)j * ldkv));
    st4(red + grp * hs + sub * 4, acc);
  }
  __syncthreads();
  if (tid < hs) {
    float o = 0.f;
    for (int g = 0; g < ngrp; ++g) o += red[g * hs + tid];
    out[(size_t)i * ldo + h * hs + tid] = o;
  }
}


// Prefill attention for head size 64 with K and V tiled through LDS: one workgroup
// per (head, block of 16 query rows). Keys are visited in tiles of 64: the K and V
// rows of the tile are staged in LDS once and shared by the 16 queries (the
// per-query kernel above re-reads every row from L2 for every query). Thread
// (q = tid/16, c = tid%16): scores of query q for keys c, c+16, c+32, c+48 of the
// tile (q row in registers, K rows from LDS), running softmax over tiles, then the
// four output columns 4c..4c+3 of query q (weights through LDS, V rows from LDS).
// Arithmetic as the reference up to re-association: scale after the dot
// (instructions.js:1176), masked keys contribute nothing, exp(x - max) / sum.
constexpr int ATQ = 16, ATK = 64, AHS = 64, AKS = AHS + 4;  // row stride of the staged tiles (bank spread)
__device__ __forceinline__ float row16_allsum(float v) {
  v += __shfl_xor(v, 8);
  v += __shfl_xor(v, 4);
  v += __shfl_xor(v, 2);
  v += __shfl_xor(v, 1);
  return v;
}
__device__ __forceinline__ float row16_allmax(float v) {
  v = fmaxf(v, __shfl_xor(v, 8));
  v = fmaxf(v, __shfl_xor(v, 4));
  v = fmaxf(v, __shfl_xor(v, 2));
  v = fmaxf(v, __shfl_xor(v, 1));
  return v;
}

__global__ __launch_bounds__(WG) void attention_tile_kernel(int Tq, int pos0, float scale, const float* __restrict__ q, int ldq,
                                                             const float* __restrict__ Kc, const float* __restrict__ Vc,
                                                             size_t hstride, int ldkv, float* __restrict__ out, int ldo) {
  __shared__ float Ks[ATK * AKS];
  __shared__ float Vs[ATK * AKS];
  __shared__ float Ps[ATQ * ATK];
  const int h = blockIdx.x, i0 = blockIdx.y * ATQ;
  const int tid = threadIdx.x, qi = tid >> 4, c = tid & 15;
  const int i = i0 + qi;                 // query row of this thread (may be >= Tq in the last block)
  const int p = pos0 + i;                // its absolute position: keys 0..p are visible
  const int pmax = pos0 + (i0 + ATQ - 1 < Tq - 1 ? i0 + ATQ - 1 : Tq - 1);
  float4 qr[AHS / 4];
#pragma unroll
  for (int k = 0; k < AHS / 4; ++k)
    qr[k] = i < Tq ? ld4(q + (size_t)i * ldq + h * AHS + 4 * k) : make_float4(0.f, 0.f, 0.f, 0.f);
  const float* kbase = Kc + h * hstride;
  const float* vbase = Vc + h * hstride;
  float m = -INFINITY, l = 0.f;
  float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int j0 = 0; j0 <= pmax; j0 += ATK) {
    __syncthreads();  // previous tile fully consumed
    // stage the tile: 64 rows x 16 float4, 256 threads x 4
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = (tid >> 4) + 16 * r, col4 = tid & 15;
      float4 kv = make_float4(0.f, 0.f, 0.f, 0.f), vv = kv;
      if (j0 + row <= pmax) {
        kv = ld4(kbase + (size_t)(j0 + row) * ldkv + 4 * col4);
        vv = ld4(vbase + (size_t)(j0 + row) * ldkv + 4 * col4);
      }
      st4(Ks + row * AKS + 4 * col4, kv);
      st4(Vs + row * AKS + 4 * col4, vv);
    }
    __syncthreads();
    // scores of keys c, c+16, c+32, c+48
    float sc[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float* kr = Ks + (c + 16 * r) * AKS;
      float a = 0.f;
#pragma unroll
      for (int k = 0; k < AHS / 4; ++k) {
        const float4 kv = ld4(kr + 4 * k);
        a += (qr[k].x * kv.x + qr[k].y * kv.y) + (qr[k].z * kv.z + qr[k].w * kv.w);
      }
      sc[r] = (j0 + c + 16 * r <= p) ? a * scale : -INFINITY;
      tmax = fmaxf(tmax, sc[r]);
    }
    tmax = row16_allmax(tmax);
    const float mnew = fmaxf(m, tmax);
    // rows beyond Tq and fully masked tiles keep m = -inf: guard the exponentials
    const float corr = mnew > -INFINITY ? expf(m - mnew) : 1.f;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float pr = sc[r] > -INFINITY ? expf(sc[r] - mnew) : 0.f;
      Ps[qi * ATK + c + 16 * r] = pr;
      psum += pr;
    }
    psum = row16_allsum(psum);
    l = l * corr + psum;
    m = mnew;
    o.x *= corr; o.y *= corr; o.z *= corr; o.w *= corr;
    __syncthreads();  // weights of the tile visible (only this query's 16 lanes wrote them, but waves differ in pace)
    const float* pr = Ps + qi * ATK;
    const float* vr = Vs + 4 * c;
#pragma unroll 8
    for (int j = 0; j < ATK; ++j) fma4(o, pr[j], ld4(vr + j * AKS));
  }
  if (i < Tq) st4(out + (size_t)i * ldo + h * AHS + 4 * c, make_float4(o.x / l, o.y / l, o.z / l, o.w / l));
}

// ---------------------------------------------------------------------------
// Prefill attention on the matrix cores (head size 64, at least 32 queries).
// A workgroup owns 32 queries of one head; its four or eight waves split the visible keys
// into contiguous runs of 32-key tiles and are merged at the end (flash-decoding).
// Everything is computed transposed, S^T = K Q^T and O^T = V^T P^T, with
// v_mfma_f32_32x32x2_f32: an accumulator then holds, per lane, 16 keys (or output
// dimensions) of ONE query (column l % 32), so the softmax over keys is a reduction
// over a lane's own registers plus one exchange with lane l ^ 32, the rescaling of
// O by exp(m_old - m_new) is a per-lane scalar, and the probabilities are already
// in the operand layout of the second product:
//   accumulator register r of lane l is row (r/4)*8 + (l/32)*4 + r%4, column l%32;
//   operand lane l supplies A[row l%32][k l/32] and B[k l/32][col l%32] per step.
// The contraction index of either product may be visited in any order as long as
// both operands agree: QK^T steps through dimension (l/32)*32 + i at step i (each
// lane's 32 dimensions are contiguous in memory), PV through key
// (i/4)*8 + (l/32)*4 + i%4 at step i (exactly the key that register i holds).
// Scores are scaled by folding 1/sqrt(hs) into Q.
// ---------------------------------------------------------------------------
constexpr int AMQ = 32;        // queries per workgroup
constexpr int AMK = 32;        // keys per tile
constexpr int AMKST = AHS + 4; // row stride of a staged K tile (conflict-free 128-bit reads by 32 rows)
constexpr int AM_WAVE_FLOATS = AMK * AMKST + AMK * AHS;  // K tile + V tile of one wave
constexpr int AMOST = AMQ + 1; // row stride of a wave's O^T[dim][query] in the merge

template <int NWV>
__global__ __launch_bounds__(NWV * 64) void attention_mfma_kernel(int Tq, int pos0, float scale, const float* __restrict__ q, int ldq,
                                                             const float* __restrict__ Kc, const float* __restrict__ Vc,
                                                             size_t hstride, int ldkv, float* __restrict__ out, int ldo) {
  extern __shared__ __attribute__((aligned(16))) float am_lds[];
  const int h = blockIdx.x, q0 = blockIdx.y * AMQ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hh = lane >> 5;
  float* Ks = am_lds + wave * AM_WAVE_FLOATS;
  float* Vs = Ks + AMK * AMKST;
  const float* kbase = Kc + h * hstride;
  const float* vbase = Vc + h * hstride;
  const int qrow = q0 + l32;                 // this lane's query (may be >= Tq in the last block)
  const int qpos = pos0 + qrow;              // keys 0..qpos are visible to it
  const int qlast = q0 + AMQ - 1 < Tq - 1 ? q0 + AMQ - 1 : Tq - 1;
  const int nkeys = pos0 + qlast + 1;        // keys any query of the block sees
  const int nt = (nkeys + AMK - 1) / AMK;
  const int per = (nt + NWV - 1) / NWV;
  const int tb = wave * per;
  const int te = tb + per < nt ? tb + per : nt;

  float qf[32];  // scaled Q[qrow][hh*32 + i]
  {
    const float* qp = q + (size_t)(qrow < Tq ? qrow : Tq - 1) * ldq + h * AHS + hh * 32;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float4 v = ld4(qp + 4 * j);
      qf[4 * j] = v.x * scale; qf[4 * j + 1] = v.y * scale; qf[4 * j + 2] = v.z * scale; qf[4 * j + 3] = v.w * scale;
    }
  }
  float m = -INFINITY, lsum = 0.f;
  f32x16 o0, o1;
#pragma unroll
  for (int r = 0; r < 16; ++r) { o0[r] = 0.f; o1[r] = 0.f; }

  // the tile after the current one is already on its way from memory while the current one is multiplied.
  // The loads are unconditional (a load under a branch is waited for where the paths join, which would undo the
  // overlap): rows past the last key repeat it; no query of the block sees them, so their weights are exactly 0
  // and the repeated values only have to be finite.
  float4 kreg[8], vreg[8];
  auto fetch = [&](int t) {
    const int k0 = t * AMK;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int f = lane + 64 * j, row = f >> 4, c4 = f & 15;
      const int key = k0 + row < nkeys ? k0 + row : nkeys - 1;
      kreg[j] = ld4(kbase + (size_t)key * ldkv + 4 * c4);
      vreg[j] = ld4(vbase + (size_t)key * ldkv + 4 * c4);
    }
  };
  fetch(tb);
  for (int t = tb; t < te; ++t) {
    const int k0 = t * AMK;
    // stage the K and V tiles of this wave: 32 rows x 16 float4 each, 8 per lane
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int f = lane + 64 * j, row = f >> 4, c4 = f & 15;
      st4(Ks + row * AMKST + 4 * c4, kreg[j]);
      st4(Vs + row * AHS + 4 * c4, vreg[j]);
    }
    fetch(t + 1);
    __builtin_amdgcn_wave_barrier();  // the tiles are private to the wave: LDS operations of a wave complete in order
    // S^T[key][query] = sum_dim K[key][dim] Q[query][dim]
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
    {
      const float* kr = Ks + l32 * AMKST + hh * 32;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float4 kv = ld4(kr + 4 * j);
        sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.x, qf[4 * j], sacc, 0, 0, 0);
        sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.y, qf[4 * j + 1], sacc, 0, 0, 0);
        sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.z, qf[4 * j + 2], sacc, 0, 0, 0);
        sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kv.w, qf[4 * j + 3], sacc, 0, 0, 0);
      }
    }
    // causal mask and the running maximum of this lane's query
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int key = k0 + (r >> 2) * 8 + hh * 4 + (r & 3);
      sacc[r] = key <= qpos ? sacc[r] : -INFINITY;
      tmax = fmaxf(tmax, sacc[r]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float mnew = fmaxf(m, tmax);
    // a query with no visible key so far keeps m = -inf: guard the exponentials
    const float corr = mnew > -INFINITY ? __expf(m - mnew) : 1.f;
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float pr = sacc[r] > -INFINITY ? __expf(sacc[r] - mnew) : 0.f;
      sacc[r] = pr;
      psum += pr;
    }
    lsum = lsum * corr + psum;
    m = mnew;
#pragma unroll
    for (int r = 0; r < 16; ++r) { o0[r] *= corr; o1[r] *= corr; }
    // O^T[dim][query] += sum_key V[key][dim] P[query][key]; step i visits the key of register i
    {
      const float* vr = Vs + hh * 4 * AHS + l32;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float* vk = vr + ((i >> 2) * 8 + (i & 3)) * AHS;
        o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(vk[0], sacc[i], o0, 0, 0, 0);
        o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(vk[32], sacc[i], o1, 0, 0, 0);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  lsum += __shfl_xor(lsum, 32);  // the two halves of a column saw disjoint keys, the same maximum

  // merge of the four waves: each leaves O^T (64 x 32), m and l of its key run in its own LDS region
  float* Om = am_lds + wave * AM_WAVE_FLOATS;  // [AHS][AMOST], then m[AMQ], l[AMQ]
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int dim = (r >> 2) * 8 + hh * 4 + (r & 3);
    Om[dim * AMOST + l32] = o0[r];
    Om[(dim + 32) * AMOST + l32] = o1[r];
  }
  if (hh == 0) {
    Om[AHS * AMOST + l32] = m;
    Om[AHS * AMOST + AMQ + l32] = lsum;
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < AMQ * AHS / (NWV * 64); ++j) {
    const int e = tid + NWV * 64 * j, qi = e >> 6, dim = e & 63;
    float mw[NWV], M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      mw[w] = am_lds[w * AM_WAVE_FLOATS + AHS * AMOST + qi];
      M = fmaxf(M, mw[w]);
    }
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) {
      const float f = mw[w] > -INFINITY ? __expf(mw[w] - M) : 0.f;
      num += am_lds[w * AM_WAVE_FLOATS + dim * AMOST + qi] * f;
      den += am_lds[w * AM_WAVE_FLOATS + AHS * AMOST + AMQ + qi] * f;
    }
    if (q0 + qi < Tq) out[(size_t)(q0 + qi) * ldo + h * AHS + dim] = num / den;
  }
}

// ---------------------------------------------------------------------------
// One decode token with one launch per block of the layer (the path of every model shape, replayable as a HIP
// graph: nothing in a launch depends on the position except through *pos).
//
// gemv_slab_kernel: FastMatMulBlock at M = 1 (instructions.js:248-314) in ONE launch and one pass. The weights
// are read from the decode slabs, in which the K values of a column are contiguous (segments of 256: 64 lanes x
// float4, or x one word of four int8; K zero-padded to S segments): a wave owns R whole columns, so a dot product
// never leaves its wave, no partial sums pass through memory and the sum has one fixed order. Every workgroup
// first builds the input row in LDS, with the LayerNormBlock in front of the product applied on the way
// (instructions.js:451-550: layernorm_kernel's order of operations; each workgroup repeats the two reductions
// over the few KB of the row rather than wait for a separate launch). fp32 slabs of c_attn and c_fc hold
// diag(gamma) W and their bias holds bias + beta W, so for them the row is only normalised (ROW_NORMALISE);
// int8 slabs take the full LayerNorm (ROW_LAYERNORM). int8 weights are dequantised one by one as the shader does,
// float(q) / 127.0f * scale[n] (other/int8-gemm.js:126-132). Bias last, then GELU or the residual add; the key
// and value columns of a q/k/v row also go to cache row *pos.
// ---------------------------------------------------------------------------
enum { ROW_PLAIN = 0, ROW_NORMALISE = 1, ROW_LAYERNORM = 2, ROW_MERGE = 3 };
struct GemvSlabArgs {
  int N, K, S;
  const void* slab;
  const float* scale;   // int8: per column
  const float* x;       // [K]
  int row_mode;
  const float* gamma;
  const float* beta;
  const float* bias;
  int epi;
  const float* resid;   // [N], may alias C
  float* C;             // [N]
  float* Kc;            // null: no cache scatter
  float* Vc;
  int d, hs, ctx;
  const int* pos;
  int nslice;           // ROW_MERGE: x holds [K / mhs][nslice][mhs + 4] attention slices, of which the first nmerge are read
  int mhs;
  int nmerge;
};

typedef float nt_f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ld4_stream(const float4* p) {  // read once per token: keep it out of the way of the row and the cache
  const nt_f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const nt_f32x4*>(p));
  return make_float4(t.x, t.y, t.z, t.w);
}

template <int R, bool I8>
__global__ __launch_bounds__(WG) void gemv_slab_kernel(GemvSlabArgs a) {
  // segments of a column requested at a time (two register sets of this many): sized so that the kernel stays within
  // 128 registers and two workgroups fit a compute unit (grids of 300-400 workgroups then run in one round)
  constexpr int CH = (!I8 && R > 1) ? 4 : 8;
  extern __shared__ __attribute__((aligned(16))) float xs[];  // [S * 256]
  __shared__ float sh[NWAVE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int k4 = a.K >> 2, s64 = a.S * 64;
  // This wave's columns (beyond N: the last one again, never stored) and the first chunk of their weights, which
  // do not depend on the row: requested before the row is built, so that they travel during the LayerNorm.
  const int col0 = (blockIdx.x * NWAVE + wave) * R;
  typedef typename std::conditional<I8, int32_t, float4>::type Item;
  const Item* base[R];
  float4 sc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int col = col0 + r < a.N ? col0 + r : a.N - 1;
    base[r] = static_cast<const Item*>(a.slab) + (size_t)col * a.S * 64 + lane;
    if (I8) {
      const float s = a.scale[col];
      sc[r] = make_float4(s, s, s, s);
    }
  }
  // What the epilogue adds is requested now as well: a load behind the dot products would be one more memory round
  // trip at the end of a kernel that consists of little else. (resid may be C itself: column n is read and written
  // by its owner only.)
  float ebias[R], eres[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int col = col0 + r < a.N ? col0 + r : a.N - 1;
    ebias[r] = a.bias ? a.bias[col] : 0.f;
    eres[r] = a.epi == EPI_RESIDUAL ? a.resid[col] : 0.f;
  }
  const int kvpos = a.Kc ? *a.pos : 0;
  // ... and the LayerNorm parameters of this thread's first two float4 of the row (int8 slabs do not carry them)
  float4 gpre[2], bpre[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    gpre[p] = bpre[p] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (a.row_mode == ROW_LAYERNORM) {
      const int i = tid + WG * p < k4 ? tid + WG * p : k4 - 1;
      gpre[p] = ld4(a.gamma + 4 * i);
      bpre[p] = ld4(a.beta + 4 * i);
    }
  }
  Item w0[R][CH], w1[R][CH];
  auto request = [&](Item (&w)[R][CH], int c0) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        // unconditional: a segment beyond S repeats the last one and meets zeros
        const int seg = c0 + j < a.S ? c0 + j : a.S - 1;
        if constexpr (I8) w[r][j] = __builtin_nontemporal_load(base[r] + (size_t)seg * 64);
        else w[r][j] = ld4_stream(base[r] + (size_t)seg * 64);
      }
  };
  request(w0, 0);

  float s1 = 0.f;
  if (a.row_mode == ROW_MERGE) {
    // the row is the attention output, still in slices of the context: (o[hs] unnormalised, max, sum) per head and
    // slice, combined here as attention_decode_slice_kernel's header describes
    const int stride = a.mhs + 4;
    for (int i = tid; i < s64; i += WG) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (i < k4) {
        const int h = (4 * i) / a.mhs, e = 4 * i - h * a.mhs;
        const float* ph = a.x + (size_t)h * a.nslice * stride;
        // eight slices at a time, everything requested before anything is used: one round trip, not one per slice
        float mx = -3.402823e+38f, den = 0.f;
        for (int s0 = 0; s0 < a.nmerge; s0 += 8) {
          float mv[8], lv[8];
          float4 ov[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int sl = s0 + j < a.nmerge ? s0 + j : a.nmerge - 1;
            mv[j] = ph[sl * stride + a.mhs];
            lv[j] = ph[sl * stride + a.mhs + 1];
            ov[j] = ld4(ph + sl * stride + e);
          }
          float mnew = mx;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (s0 + j < a.nmerge) mnew = fmaxf(mnew, mv[j]);
          const float keep = expf(mx - mnew);  // rescales what earlier groups of eight have left
          den *= keep;
          v = make_float4(v.x * keep, v.y * keep, v.z * keep, v.w * keep);
          mx = mnew;
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (s0 + j < a.nmerge) {
              const float w = expf(mv[j] - mx);
              den += w * lv[j];
              fma4(v, w, ov[j]);
            }
        }
        v = make_float4(v.x / den, v.y / den, v.z / den, v.w / den);
      }
      st4(xs + 4 * i, v);
    }
  } else {
    for (int i = tid; i < s64; i += WG) {
      const float4 v = i < k4 ? ld4(a.x + 4 * i) : make_float4(0.f, 0.f, 0.f, 0.f);
      st4(xs + 4 * i, v);
      s1 += (v.x + v.y) + (v.z + v.w);
    }
  }
  if (a.row_mode == ROW_NORMALISE || a.row_mode == ROW_LAYERNORM) {
    const float mean = block_sum(s1, sh) / (float)a.K;
    float q = 0.f;
    for (int i = tid; i < k4; i += WG) {
      const float4 v = ld4(xs + 4 * i);
      const float e0 = v.x - mean, e1 = v.y - mean, e2 = v.z - mean, e3 = v.w - mean;
      q += (e0 * e0 + e1 * e1) + (e2 * e2 + e3 * e3);
    }
    const float var = block_sum(q, sh) / (float)a.K;
    const float stdev = sqrtf(var + 1e-5f);
    for (int i = tid, p = 0; i < k4; i += WG, ++p) {
      const float4 v = ld4(xs + 4 * i);
      float4 o = make_float4((v.x - mean) / stdev, (v.y - mean) / stdev, (v.z - mean) / stdev, (v.w - mean) / stdev);
      if (a.row_mode == ROW_LAYERNORM) {
        const float4 g = p == 0 ? gpre[0] : (p == 1 ? gpre[1] : ld4(a.gamma + 4 * i));
        const float4 b = p == 0 ? bpre[0] : (p == 1 ? bpre[1] : ld4(a.beta + 4 * i));
        o = make_float4(g.x * o.x + b.x, g.y * o.y + b.y, g.z * o.z + b.z, g.w * o.w + b.w);
      }
      st4(xs + 4 * i, o);
    }
  }
  __syncthreads();
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.f;
  auto contract = [&](const Item (&w)[R][CH], int c0) {
#pragma unroll
    for (int j = 0; j < CH; ++j) {
      float4 xv = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c0 + j < a.S) xv = ld4(xs + (c0 + j) * 256 + lane * 4);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float4 wv;
        if constexpr (I8) wv = unpack_i8x4_k(w[r][j], sc[r]);
        else wv = w[r][j];
        acc[r] += (wv.x * xv.x + wv.y * xv.y) + (wv.z * xv.z + wv.w * xv.w);
      }
    }
  };
  for (int c0 = 0; c0 < a.S; c0 += 2 * CH) {
    if (c0 + CH < a.S) request(w1, c0 + CH);
    contract(w0, c0);
    if (c0 + CH < a.S) {
      if (c0 + 2 * CH < a.S) request(w0, c0 + 2 * CH);
      contract(w1, c0 + CH);
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float v = wave_sum(acc[r]);
    const int n = col0 + r;
    if (lane == 0 && n < a.N) {
      if (a.bias) v += ebias[r];
      if (a.epi == EPI_GELU) v = gelu_ref(v);
      else if (a.epi == EPI_RESIDUAL) v += eres[r];
      a.C[n] = v;
      if (a.Kc && n >= a.d) {
        const int which = n >= 2 * a.d, c = n - (1 + which) * a.d, h = c / a.hs, e = c - h * a.hs;
        (which ? a.Vc : a.Kc)[((size_t)h * a.ctx + kvpos) * a.hs + e] = v;
      }
    }
  }
}

// Attention of ONE query (the token being decoded, at cache position *pos) per head: formatQ + fusedWeights +
// softmax + attentionValues of instructions.js:1129-1212 as attention_kernel computes them, arranged for the
// latency of a single dependent chain: a workgroup per head requests the first 16 key rows AND value rows of each
// of its lane groups (256 positions at head size 64) before anything else, so a context of up to 256 positions
// costs one memory round trip; longer contexts continue in batches of the same size.
__global__ __launch_bounds__(WG) void attention_decode_kernel(int hs, int lpk, int ctx, float scale, const float* __restrict__ q,
                                                               const float* __restrict__ Kc, const float* __restrict__ Vc,
                                                               size_t hstride, float* __restrict__ out, const int* __restrict__ pos) {
  constexpr int U = 16;
  extern __shared__ __attribute__((aligned(16))) float scores[];
  __shared__ float red[1024];
  __shared__ float sh[NWAVE];
  const int h = blockIdx.x, tid = threadIdx.x;
  const int sub = tid & (lpk - 1), grp = tid / lpk, ngrp = WG / lpk;
  const bool act = sub * 4 < hs;
  const float* kbase = Kc + h * hstride + (act ? sub * 4 : 0);
  const float* vbase = Vc + h * hstride + (act ? sub * 4 : 0);
  // The first batch is requested before the position is known (rows up to the end of the cache exist; those
  // beyond the context hold finite leftovers and are not used): its round trip overlaps that of *pos.
  const float4 qv = act ? ld4(q + h * hs + sub * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
  float4 k0[U], v0[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int j = u * ngrp + grp;
    j = j < ctx ? j : ctx - 1;
    k0[u] = ld4(kbase + (size_t)j * hs);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int j = u * ngrp + grp;
    j = j < ctx ? j : ctx - 1;
    v0[u] = ld4(vbase + (size_t)j * hs);
  }
  const int nkeys = *pos + 1;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int j = u * ngrp + grp;
    float part = (qv.x * k0[u].x + qv.y * k0[u].y) + (qv.z * k0[u].z + qv.w * k0[u].w);
    for (int off = lpk >> 1; off > 0; off >>= 1) part += __shfl_xor(part, off);
    if (sub == 0 && j < nkeys) scores[j] = part * scale;
  }
  for (int j0 = U * ngrp; j0 < nkeys; j0 += U * ngrp) {
    float4 kv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int j = j0 + u * ngrp + grp;
      j = j < nkeys ? j : nkeys - 1;
      kv[u] = ld4(kbase + (size_t)j * hs);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * ngrp + grp;
      float part = (qv.x * kv[u].x + qv.y * kv[u].y) + (qv.z * kv[u].z + qv.w * kv[u].w);
      for (int off = lpk >> 1; off > 0; off >>= 1) part += __shfl_xor(part, off);
      if (sub == 0 && j < nkeys) scores[j] = part * scale;
    }
  }
  __syncthreads();
  float m = -3.402823e+38f;
  for (int j = tid; j < nkeys; j += WG) m = fmaxf(m, scores[j]);
  m = block_max(m, sh);
  float s = 0.f;
  for (int j = tid; j < nkeys; j += WG) {
    const float e = expf(scores[j] - m);
    scores[j] = e;
    s += e;
  }
  s = block_sum(s, sh);
  for (int j = tid; j < nkeys; j += WG) scores[j] = scores[j] / s;
  __syncthreads();
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int j = u * ngrp + grp;
    if (j < nkeys) fma4(acc, scores[j], v0[u]);
  }
  for (int j0 = U * ngrp; j0 < nkeys; j0 += U * ngrp) {
    float4 vv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int j = j0 + u * ngrp + grp;
      j = j < nkeys ? j : nkeys - 1;
      vv[u] = ld4(vbase + (size_t)j * hs);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = j0 + u * ngrp + grp;
      if (j < nkeys) fma4(acc, scores[j], vv[u]);
    }
  }
  if (act) st4(red + grp * hs + sub * 4, acc);
  __syncthreads();
  if (tid < hs) {
    float o = 0.f;
    for (int g = 0; g < ngrp; ++g) o += red[g * hs + tid];
    out[h * hs + tid] = o;
  }
}

// The same attention with the cache cut into fixed slices of ADS_ROWS x WG / lanes-per-key positions (64 at head size
// 64), a workgroup per (head, slice): the rows of a slice are one small request per lane group, so a context of any
// length is one memory round trip, spread over as many compute units as it has slices (one workgroup per head
// streaming a whole context is bound by what a single compute unit can fetch: 10 us at 150 positions, 25 us at 550).
// A slice up to the position the caller expects (spec_pos, the host's knowledge of *pos) requests its rows before it
// has read *pos; the others read *pos first and leave at once if they lie beyond the context. A slice leaves
// (sum_j e_j v_j, m, sum_j e_j) with e_j = exp(score_j - m), m its own maximum (flash-decoding); one beyond the
// context leaves (0, -FLT_MAX, 0). The consumer (gemv_slab_kernel, ROW_MERGE) combines them:
// out = sum_s w_s o_s / sum_s w_s l_s with w_s = exp(m_s - max_s m_s), which is softmax(scores) . V of
// instructions.js:1129-1212 in another order of summation.
constexpr int ADS_ROWS = 4;
__global__ __launch_bounds__(WG) void attention_decode_slice_kernel(int hs, int lpk, int ctx, float scale, const float* __restrict__ q,
                                                                     const float* __restrict__ Kc, const float* __restrict__ Vc,
                                                                     size_t hstride, float* __restrict__ part, const int* __restrict__ pos,
                                                                     int spec_pos) {
  constexpr int U = ADS_ROWS;
  extern __shared__ __attribute__((aligned(16))) float scores[];  // [U * WG / lpk]
  __shared__ float red[1024];
  __shared__ float sh[NWAVE];
  const int h = blockIdx.x, sl = blockIdx.y, nsl = gridDim.y, tid = threadIdx.x;
  const int sub = tid & (lpk - 1), grp = tid / lpk, ngrp = WG / lpk;
  const int j_lo = sl * U * ngrp;
  const bool act = sub * 4 < hs;
  const float* kbase = Kc + h * hstride + (act ? sub * 4 : 0);
  const float* vbase = Vc + h * hstride + (act ? sub * 4 : 0);
  // An expected slice requests its rows before the position is known (rows up to the end of the cache exist), as
  // attention_decode_kernel does. The others look at the position first: most of them are beyond the context most of
  // the time, and their rows would be most of the launch's traffic for nothing.
  const float4 qv = act ? ld4(q + h * hs + sub * 4) : make_float4(0.f, 0.f, 0.f, 0.f);  // (first: nothing below may wait for it)
  const bool spec = j_lo <= spec_pos;  // the caller expects this slice to have positions
  int n_here = 0;
  if (!spec) n_here = min(*pos + 1 - j_lo, U * ngrp);
  float* dst = part + ((size_t)h * nsl + sl) * (hs + 4);
  if (!spec && n_here <= 0) {
    if (tid < hs) dst[tid] = 0.f;
    if (tid == 0) {
      dst[hs] = -3.402823e+38f;
      dst[hs + 1] = 0.f;
    }
    return;
  }
  float4 k0[U], v0[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int j = j_lo + u * ngrp + grp;
    j = j < ctx ? j : ctx - 1;
    k0[u] = ld4(kbase + (size_t)j * hs);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    int j = j_lo + u * ngrp + grp;
    j = j < ctx ? j : ctx - 1;
    v0[u] = ld4(vbase + (size_t)j * hs);
  }
  if (spec) {
    n_here = min(*pos + 1 - j_lo, U * ngrp);  // positions of this slice inside the context
    if (n_here <= 0) {                        // (the caller's expectation was wrong)
      if (tid < hs) dst[tid] = 0.f;
      if (tid == 0) {
        dst[hs] = -3.402823e+38f;
        dst[hs + 1] = 0.f;
      }
      return;
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int jl = u * ngrp + grp;
    float p = (qv.x * k0[u].x + qv.y * k0[u].y) + (qv.z * k0[u].z + qv.w * k0[u].w);
    for (int off = lpk >> 1; off > 0; off >>= 1) p += __shfl_xor(p, off);
    if (sub == 0 && jl < n_here) scores[jl] = p * scale;
  }
  __syncthreads();
  float m = -3.402823e+38f;
  for (int j = tid; j < n_here; j += WG) m = fmaxf(m, scores[j]);
  m = block_max(m, sh);
  float l = 0.f;
  for (int j = tid; j < n_here; j += WG) {
    const float e = expf(scores[j] - m);
    scores[j] = e;
    l += e;
  }
  l = block_sum(l, sh);
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int jl = u * ngrp + grp;
    if (jl < n_here) fma4(acc, scores[jl], v0[u]);
  }
  if (act) st4(red + grp * hs + sub * 4, acc);
  __syncthreads();
  if (tid < hs) {
    float o = 0.f;
    for (int g = 0; g < ngrp; ++g) o += red[g * hs + tid];
    dst[tid] = o;
  }
  if (tid == 0) {
    dst[hs] = m;
    dst[hs + 1] = l;
  }
}

// The final LayerNormBlock (model.js:224) and DeEmbedBlock (instructions.js:916-943) of a decode token in one
// launch: every workgroup normalises the row itself while staging it (layernorm_kernel's order of operations), then
// vocab_gemv_kernel's rows; the first workgroup finally advances the cache position, if the caller passes one (nothing
// later in the token reads it).
__global__ __launch_bounds__(WG) void vocab_gemv_ln_kernel(int V, int d, const float* __restrict__ x, const float* __restrict__ gamma,
                                                            const float* __restrict__ beta, const float* __restrict__ wte,
                                                            float* __restrict__ logits, int* pos) {
  extern __shared__ __attribute__((aligned(16))) float xs[];
  __shared__ float sh[NWAVE];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int v0 = (blockIdx.x * NWAVE + wave) * VOCAB_ROWS_PER_WAVE;
  const int n4 = d >> 2;
  // Everything that does not depend on the row is requested first, so that it travels during the LayerNorm: the first
  // two sweeps of this wave's table rows, and the LayerNorm parameters of this thread's first two float4 of the row.
  constexpr int PRE = 2;
  float4 wpre[PRE][VOCAB_ROWS_PER_WAVE], gpre[PRE], bpre[PRE];
#pragma unroll
  for (int p = 0; p < PRE; ++p) {
    const int c = lane + 64 * p < n4 ? lane + 64 * p : n4 - 1;
#pragma unroll
    for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) {
      const int row = v0 + r < V ? v0 + r : V - 1;
      wpre[p][r] = ld4(wte + (size_t)row * d + 4 * c);
    }
    const int ct = (int)threadIdx.x + WG * p < n4 ? (int)threadIdx.x + WG * p : n4 - 1;
    gpre[p] = ld4(gamma + 4 * ct);
    bpre[p] = ld4(beta + 4 * ct);
  }
  float s1 = 0.f;
  for (int c = threadIdx.x; c < n4; c += WG) {
    const float4 v = ld4(x + 4 * c);
    st4(xs + 4 * c, v);
    s1 += (v.x + v.y) + (v.z + v.w);
  }
  const float mean = block_sum(s1, sh) / (float)d;
  float q = 0.f;
  for (int c = threadIdx.x; c < n4; c += WG) {
    const float4 v = ld4(xs + 4 * c);
    const float e0 = v.x - mean, e1 = v.y - mean, e2 = v.z - mean, e3 = v.w - mean;
    q += (e0 * e0 + e1 * e1) + (e2 * e2 + e3 * e3);
  }
  const float var = block_sum(q, sh) / (float)d;
  const float stdev = sqrtf(var + 1e-5f);
  for (int c = threadIdx.x, p = 0; c < n4; c += WG, ++p) {
    const float4 v = ld4(xs + 4 * c);
    const float4 g = p == 0 ? gpre[0] : (p == 1 ? gpre[1] : ld4(gamma + 4 * c));
    const float4 b = p == 0 ? bpre[0] : (p == 1 ? bpre[1] : ld4(beta + 4 * c));
    st4(xs + 4 * c, make_float4(g.x * ((v.x - mean) / stdev) + b.x, g.y * ((v.y - mean) / stdev) + b.y,
                                g.z * ((v.z - mean) / stdev) + b.z, g.w * ((v.w - mean) / stdev) + b.w));
  }
  __syncthreads();
  float acc[VOCAB_ROWS_PER_WAVE];
#pragma unroll
  for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) acc[r] = 0.f;
#pragma unroll
  for (int p = 0; p < PRE; ++p) {
    const int c = lane + 64 * p;
    if (c < n4) {
      const float4 xv = ld4(xs + 4 * c);
#pragma unroll
      for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) {
        const float4 w = wpre[p][r];
        if (v0 + r < V) acc[r] += (xv.x * w.x + xv.y * w.y) + (xv.z * w.z + xv.w * w.w);
      }
    }
  }
  for (int c = lane + 64 * PRE; c < n4; c += 64) {
    const float4 xv = ld4(xs + 4 * c);
#pragma unroll
    for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) {
      if (v0 + r < V) {
        const float4 w = ld4(wte + (size_t)(v0 + r) * d + 4 * c);
        acc[r] += (xv.x * w.x + xv.y * w.y) + (xv.z * w.z + xv.w * w.w);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < VOCAB_ROWS_PER_WAVE; ++r) {
    const float sum = wave_sum(acc[r]);
    if (lane == 0 && v0 + r < V) logits[v0 + r] = sum;
  }
  if (pos && blockIdx.x == 0 && threadIdx.x == 0) *pos += 1;
}


__global__ __launch_bounds__(WG) void copy_rows_kernel(int cols4, const float* __restrict__ src, int lds,
                                                        float* __restrict__ dst, int ldd) {
  const int r = blockIdx.y;
  const int c = blockIdx.x * WG + threadIdx.x;
  if (c < cols4) st4(dst + (size_t)r * ldd + 4 * c, ld4(src + (size_t)r * lds + 4 * c));
}

// Appends T rows of keys and values (columns d..2d and 2d..3d of qkv[T,3d]) to the
// head-major cache: row (h, pos0+i) of K at Kc + (h*ctx + pos0+i)*hs.
__global__ __launch_bounds__(WG) void kv_append_kernel(int d, int hs, int ctx, int pos0, const float* __restrict__ qkv,
                                                        float* __restrict__ Kc, float* __restrict__ Vc) {
  const int i = blockIdx.x;
  for (int c4 = threadIdx.x; c4 < (d >> 2); c4 += WG) {
    const int c = c4 * 4, h = c / hs, e = c - h * hs;
    const size_t dst = ((size_t)h * ctx + pos0 + i) * hs + e;
    st4(Kc + dst, ld4(qkv + (size_t)i * 3 * d + d + c));
    st4(Vc + dst, ld4(qkv + (size_t)i * 3 * d + 2 * d + c));
  }
}

// Token selection of GPT.generate (model.js:81-85) on the device, one workgroup:
//   selectTopK (globals.js:66-74): stable descending sort of (value, index), first k;
//     here k rounds of arg-max with the lowest index among equal values;
//   cpuSoftmax (globals.js:59-64) of those k logits in float64:
//     exp((x - max) / temperature), summed left to right, divided by the sum;
//   sampleFromDistribution (globals.js:47-57): first i with u < p_0 + .. + p_i, else k - 1;
//     u is the caller's uniform draw in [0, 1) (the reference's Math.random()).
// The chosen id goes to tok[0] (input of the next decode step) and out[slot]; ids/probs
// (optional) receive the k selected indices and their probabilities.
__device__ __forceinline__ bool better(float ov, int oi, float cv, int ci) {
  return oi != 0x7fffffff && (ci == 0x7fffffff || ov > cv || (ov == cv && oi < ci));
}

// REG: the logits of a thread's stride (V <= 65536: at most 64 of them) stay in registers, so the
// owner's search for its next candidate after a selection touches no memory.
template <bool REG>
__global__ __launch_bounds__(1024) void sample_topk_kernel(int V, int k, double temperature, const double* __restrict__ u,
                                                            const float* __restrict__ logits, int32_t* tok, int32_t* out, int slot,
                                                            int32_t* ids, double* probs) {
  __shared__ unsigned taken[SAMPLE_MAX_V / 32];
  __shared__ float wv[16];
  __shared__ int wi[16];
  __shared__ float sel_v[SAMPLE_MAX_K];
  __shared__ int sel_i[SAMPLE_MAX_K];
  __shared__ double ev[SAMPLE_MAX_K];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (!REG)
    for (int i = tid; i < (V + 31) / 32; i += 1024) taken[i] = 0u;
  if (k > V) k = V;
  float mine[REG ? 64 : 1];
  unsigned long long gone = 0ull;  // REG: bit j set once element tid + 1024 j has been selected
  if (REG) {
#pragma unroll
    for (int j = 0; j < 64; ++j) mine[j] = tid + 1024 * j < V ? logits[tid + 1024 * j] : -INFINITY;
  }
  // this thread's candidate: the best not yet taken element of its stride
  auto scan = [&](float& best, int& besti) {
    best = -INFINITY;
    besti = 0x7fffffff;
    if (REG) {
#pragma unroll
      for (int j = 0; j < 64; ++j) {
        const int i = tid + 1024 * j;
        if (i < V && !((gone >> j) & 1ull) && (mine[REG ? j : 0] > best || besti == 0x7fffffff)) {
          best = mine[REG ? j : 0];
          besti = i;
        }
      }
      return;
    }
    for (int i = tid; i < V; i += 1024) {
      if (taken[i >> 5] & (1u << (i & 31))) continue;
      const float v = logits[i];
      if (v > best || besti == 0x7fffffff) {
        best = v;
        besti = i;
      }
    }
  };
  __syncthreads();
  float best;
  int besti;
  scan(best, besti);
  for (int r = 0; r < k; ++r) {
    float cv = best;
    int ci = besti;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(cv, off);
      const int oi = __shfl_xor(ci, off);
      if (better(ov, oi, cv, ci)) {
        cv = ov;
        ci = oi;
      }
    }
    if (lane == 0) {
      wv[wave] = cv;
      wi[wave] = ci;
    }
    __syncthreads();
    cv = wv[0];
    ci = wi[0];
#pragma unroll
    for (int w = 1; w < 16; ++w)
      if (better(wv[w], wi[w], cv, ci)) {
        cv = wv[w];
        ci = wi[w];
      }
    // every thread knows the winner; its owner marks it and looks for its next candidate
    if (tid == 0) {
      sel_v[r] = cv;
      sel_i[r] = ci;
    }
    if ((ci & 1023) == tid) {
      if (REG) gone |= 1ull << (ci >> 10);
      else taken[ci >> 5] |= 1u << (ci & 31);
      scan(best, besti);
    }
    __syncthreads();
  }
  if (tid == 0) {
    const double mx = (double)sel_v[0];
    double sum = 0.0;
    for (int i = 0; i < k; ++i) {
      ev[i] = exp(((double)sel_v[i] - mx) / temperature);
      sum += ev[i];
    }
    const double rnd = *u;
    double cum = 0.0;
    int pick = k - 1;
    bool found = false;
    for (int i = 0; i < k; ++i) {
      const double p = ev[i] / sum;
      if (probs) probs[i] = p;
      if (ids) ids[i] = sel_i[i];
      cum += p;
      if (!found && rnd < cum) {
        pick = i;
        found = true;
      }
    }
    tok[0] = sel_i[pick];
    if (out) out[slot] = sel_i[pick];
  }
}

// Greedy selection: selectTopK with top_k = 1 (globals.js:66-74) is a stable
// descending sort, i.e. the largest logit with the lowest index on ties.
__global__ __launch_bounds__(1024) void argmax_kernel(int V, const float* __restrict__ logits, int32_t* tok, int32_t* out,
                                                       int slot) {
  __shared__ float bv[1024];
  __shared__ int bi[1024];
  float best = -INFINITY;
  int besti = 0x7fffffff;
  // eight loads in flight per thread (one after the other, V = 50257 took 16 us); ascending i, so ties keep the lowest index
  for (int i0 = threadIdx.x; i0 < V; i0 += 8 * 1024) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = i0 + u * 1024 < V ? logits[i0 + u * 1024] : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * 1024;
      if (i < V && (v[u] > best || besti == 0x7fffffff)) {
        best = v[u];
        besti = i;
      }
    }
  }
  bv[threadIdx.x] = best;
  bi[threadIdx.x] = besti;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) {
      const float ov = bv[threadIdx.x + s];
      const int oi = bi[threadIdx.x + s];
      const float cv = bv[threadIdx.x];
      const int ci = bi[threadIdx.x];
      if (oi != 0x7fffffff && (ci == 0x7fffffff || ov > cv || (ov == cv && oi < ci))) {
        bv[threadIdx.x] = ov;
        bi[threadIdx.x] = oi;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    tok[0] = bi[0];
    if (out) out[slot] = bi[0];
  }
}

inline unsigned cdiv(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace

// second pass of a matrix-vector product: slices side by side (up to sixteen slices the sum is still in ascending order)
static void launch_gemv_reduce(int M, int N, int S, const float* workspace, const float* bias, float* C, int ldc, int epi,
                               const float* resid, hipStream_t s) {
  if (S >= 4) gemv_reduce_wide<<<cdiv((size_t)M * (N >> 2), 16), WG, 0, s>>>(M, N, S, workspace, bias, C, ldc, epi, resid);
  else gemv_reduce<<<cdiv((size_t)M * (N >> 2), WG), WG, 0, s>>>(M, N, S, workspace, bias, C, ldc, epi, resid);
}

size_t gemv_workspace_floats(int M, int N, int K) {
  return (size_t)cdiv(K, GEMV_KCHUNK) * (size_t)(M < 1 ? 1 : M) * (size_t)N;
}

hipError_t launch_gemv_kn(int M, int N, int K, const float* A, int lda, const float* W, int ldw, const float* bias,
                          float* C, int ldc, int epi, const float* resid, float* workspace, hipStream_t s) {
  const int S = cdiv(K, GEMV_KCHUNK);
  const dim3 grid(cdiv(N, 64), S);
  switch (M) {
    case 1: gemv_kn_partial<1><<<grid, WG, 0, s>>>(N, K, A, lda, W, ldw, workspace); break;
    case 2: gemv_kn_partial<2><<<grid, WG, 0, s>>>(N, K, A, lda, W, ldw, workspace); break;
    case 3: gemv_kn_partial<3><<<grid, WG, 0, s>>>(N, K, A, lda, W, ldw, workspace); break;
    case 4: gemv_kn_partial<4><<<grid, WG, 0, s>>>(N, K, A, lda, W, ldw, workspace); break;
    default: return hipErrorInvalidValue;
  }
  launch_gemv_reduce(M, N, S, workspace, bias, C, ldc, epi, resid, s);
  return hipGetLastError();
}

hipError_t launch_gemv_kn_i8(int M, int N, int K, const float* A, int lda, const int32_t* Wq, int ldwq,
                             const float* scale, const float* bias, float* C, int ldc, int epi, const float* resid,
                             float* workspace, hipStream_t s) {
  const int S = cdiv(K, GEMV_KCHUNK);
  const dim3 grid(cdiv(N, 256), S);
  switch (M) {
    case 1: gemv_kn_i8_partial<1><<<grid, WG, 0, s>>>(N, K, A, lda, Wq, ldwq, scale, workspace); break;
    case 2: gemv_kn_i8_partial<2><<<grid, WG, 0, s>>>(N, K, A, lda, Wq, ldwq, scale, workspace); break;
    case 3: gemv_kn_i8_partial<3><<<grid, WG, 0, s>>>(N, K, A, lda, Wq, ldwq, scale, workspace); break;
    case 4: gemv_kn_i8_partial<4><<<grid, WG, 0, s>>>(N, K, A, lda, Wq, ldwq, scale, workspace); break;
    default: return hipErrorInvalidValue;
  }
  launch_gemv_reduce(M, N, S, workspace, bias, C, ldc, epi, resid, s);
  return hipGetLastError();
}

hipError_t launch_dequant_i8(int K, int N, const int32_t* Wq, int ldwq, const float* scale, float* W, int ldw, hipStream_t s) {
  dequant_i8_kernel<<<cdiv((size_t)K * (N >> 2), WG), WG, 0, s>>>(K, N, Wq, ldwq, scale, W, ldw);
  return hipGetLastError();
}

size_t gemm_workspace_floats(int M, int N) { return (size_t)8 * M * N; }

namespace {
// Second pass of a split-K product: ordered sum of the S partial matrices, bias, epilogue; with `ln` the
// LayerNorm of the finished rows in the same kernel.
void finish_split(int M, int N, int S, const float* workspace, const float* bias, float* C, int ldc, int epi, const float* resid,
                  const LnAfter* ln, const KvAfter* kv, hipStream_t s) {
  if (kv) {
    gemv_reduce<<<cdiv((size_t)M * (N >> 2), WG), WG, 0, s>>>(M, N, S, workspace, bias, C, ldc, epi, resid, *kv);
    if (ln) layernorm_kernel<<<M, WG, 0, s>>>(N, C, ldc, ln->gamma, ln->beta, ln->out, ln->ldo);
    return;
  }
  if (ln && (N & 3) == 0 && N <= 4 * WG * REDUCE_LN_MAXV) {
    reduce_ln_kernel<<<M, WG, 0, s>>>(M, N, S, workspace, bias, C, ldc, epi, resid, ln->gamma, ln->beta, ln->out, ln->ldo);
    return;
  }
  gemv_reduce<<<cdiv((size_t)M * (N >> 2), WG), WG, 0, s>>>(M, N, S, workspace, bias, C, ldc, epi, resid);
  if (ln) layernorm_kernel<<<M, WG, 0, s>>>(N, C, ldc, ln->gamma, ln->beta, ln->out, ln->ldo);
}

// The same two follow-ups after a product that wrote C itself.
void finish_direct(int M, int N, const float* C, int ldc, const LnAfter* ln, const KvAfter* kv, hipStream_t s) {
  if (kv) kv_append_kernel<<<M, WG, 0, s>>>(kv->d, kv->hs, kv->ctx, kv->pos0, C, kv->Kc, kv->Vc);
  if (ln) layernorm_kernel<<<M, WG, 0, s>>>(N, C, ldc, ln->gamma, ln->beta, ln->out, ln->ldo);
}

template <int TM, int TN, int BK, bool I8W>
void run_gemm_mfma(int M, int N, int K, int S, const float* A, int lda, const void* W, int ldw, const float* wscale,
                   const float* bias, float* C, int ldc, int epi, const float* resid, float* workspace, const LnAfter* ln,
                   const KvAfter* kv, hipStream_t s) {
  const dim3 grid(cdiv(N, TN), cdiv(M, TM), S);
  // partial sums of the K slices are combined in ascending order by gemv_reduce (deterministic), bias last
  const int kchunk = S == 1 ? K : (int)cdiv(cdiv(K, S), BK) * BK;
  const bool exact = K % BK == 0;  // then every slice is whole steps (kchunk is a multiple of BK)
  const float* kb = S == 1 ? bias : nullptr;
  float* kc = S == 1 ? C : workspace;
  const int kldc = S == 1 ? ldc : N, kepi = S == 1 ? epi : EPI_NONE;
  const float* kres = S == 1 ? resid : nullptr;
  if (exact) gemm_mfma<TM, TN, BK, I8W, true><<<grid, WG, 0, s>>>(M, N, K, kchunk, A, lda, W, ldw, wscale, kb, kc, kldc, kepi, kres);
  else gemm_mfma<TM, TN, BK, I8W, false><<<grid, WG, 0, s>>>(M, N, K, kchunk, A, lda, W, ldw, wscale, kb, kc, kldc, kepi, kres);
  if (S > 1) finish_split(M, N, S, workspace, bias, C, ldc, epi, resid, ln, kv, s);
  else finish_direct(M, N, C, ldc, ln, kv, s);
}

// 128x128 tiles when they alone fill the 256 compute units twice over, else 64x64 (measured
// best or within 3 % of it from 128 to 1024 rows); then split K (at most 8 ways, slices of
// at least 128) until there are two workgroups per compute unit.
template <bool I8W>
void run_gemm(int M, int N, int K, const float* A, int lda, const void* W, int ldw, const float* wscale, const float* bias,
              float* C, int ldc, int epi, const float* resid, float* workspace, const LnAfter* ln, const KvAfter* kv,
              hipStream_t s) {
  // 64 x 128 tiles of the two-group kernel when, with K split at most 4 ways, they give each of the 256
  // compute units one workgroup (and at most two)
  const size_t pp = (size_t)cdiv(M, 64) * cdiv(N, 128);
  if (!I8W && K % PP_BK == 0 && pp >= 64) {
    int S = 1;
    while (workspace && S < 4 && pp * S < 256 && K / (2 * S) >= 128 && (K / (2 * S)) % PP_BK == 0) S *= 2;
    // whole rounds of 256 workgroups, or nearly: a last round that leaves compute units idle costs as much as a full one
    const size_t wgs = pp * S, rounds = cdiv(wgs, 256);
    if (wgs * 100 >= rounds * 256 * 85 && wgs <= 1024) {
      static const bool raised = [] {
        return hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_pingpong<PP_BK>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)PP_LDS) == hipSuccess;
      }();
      if (raised) {
        const dim3 grid(cdiv(N, 128), cdiv(M, 64), S);
        const float* Wf = static_cast<const float*>(W);
        if (S == 1) {
          gemm_pingpong<PP_BK><<<grid, PP_THREADS, PP_LDS, s>>>(M, N, K, K, A, lda, Wf, ldw, bias, C, ldc, epi, resid);
          finish_direct(M, N, C, ldc, ln, kv, s);
        } else {
          gemm_pingpong<PP_BK><<<grid, PP_THREADS, PP_LDS, s>>>(M, N, K, K / S, A, lda, Wf, ldw, nullptr, workspace, N, EPI_NONE, nullptr);
          finish_split(M, N, S, workspace, bias, C, ldc, epi, resid, ln, kv, s);
        }
        return;
      }
    }
  }
  const bool big = (size_t)cdiv(M, 128) * cdiv(N, 128) >= 512;
  const int t = big ? 128 : 64;
  constexpr int BKS = 32;  // K step of gemm_mfma
  int S = 1;
  const size_t tiles = (size_t)cdiv(M, t) * cdiv(N, t);
  while (workspace && S < 8 && tiles * S < 512 && K / (2 * S) >= 128) S *= 2;
  if (workspace && M <= 448 && tiles <= 256) {
    // Few rows: the workgroups of a launch all start together, one to a compute unit and a second one on some once
    // there are more than 256 of them, and the launch lasts as long as the busiest unit. Any slice count that
    // leaves whole K steps will do (three slices of c_attn at 128 rows are 216 workgroups of 8 steps, where four
    // are 288 of 6, two of them on 32 units): the cheapest of rounds x (steps per slice + 4 for a round's prologue
    // and epilogue). 117M T = 128: 0.895 -> 0.86 ms, T = 192: 1.07 -> 0.97; 1.5B T = 128: 6.67 -> 5.96; beyond
    // ~450 rows several workgroups share a unit anyway and the doubling rule above measures better (T = 960:
    // 2.56 against 2.63 ms).
    long best = -1;
    for (int c = 1; c <= 8; ++c) {
      if (K % (BKS * c) != 0 || (c > 1 && K / c < 96)) continue;
      const long cost = (long)cdiv(tiles * c, 256) * (K / (BKS * c) + 4);
      if (best < 0 || cost < best) {
        best = cost;
        S = c;
      }
    }
  }
  if (big) run_gemm_mfma<128, 128, 32, I8W>(M, N, K, S, A, lda, W, ldw, wscale, bias, C, ldc, epi, resid, workspace, ln, kv, s);
  else run_gemm_mfma<64, 64, 32, I8W>(M, N, K, S, A, lda, W, ldw, wscale, bias, C, ldc, epi, resid, workspace, ln, kv, s);
}
}  // namespace

hipError_t launch_gemm(int M, int N, int K, const float* A, int lda, const float* W, int ldw, const float* bias,
                       float* C, int ldc, int epi, const float* resid, float* workspace, hipStream_t s, const LnAfter* ln,
                       const KvAfter* kv) {
  if (M < 16) {
    // too few rows for a matrix-core tile: scalar-FMA tile kernel
    gemm_tile64<<<dim3(cdiv(N, 64), cdiv(M, 64)), WG, 0, s>>>(M, N, K, A, lda, W, ldw, bias, C, ldc, epi, resid);
    finish_direct(M, N, C, ldc, ln, kv, s);
    return hipGetLastError();
  }
  run_gemm<false>(M, N, K, A, lda, W, ldw, nullptr, bias, C, ldc, epi, resid, workspace, ln, kv, s);
  return hipGetLastError();
}

hipError_t launch_gemm_i8(int M, int N, int K, const float* A, int lda, const int32_t* Wq, int ldwq, const float* scale,
                          const float* bias, float* C, int ldc, int epi, const float* resid, float* workspace, hipStream_t s,
                          const LnAfter* ln, const KvAfter* kv) {
  if (M < 16 || (N & 3)) return hipErrorInvalidValue;
  run_gemm<true>(M, N, K, A, lda, Wq, ldwq, scale, bias, C, ldc, epi, resid, workspace, ln, kv, s);
  return hipGetLastError();
}

hipError_t launch_residual(size_t n4, const float* a, const float* b, float* out, hipStream_t s) {
  residual_kernel<<<cdiv(n4, WG), WG, 0, s>>>(n4, a, b, out);
  return hipGetLastError();
}

hipError_t launch_gelu(size_t n4, const float* x, float* out, hipStream_t s) {
  gelu_kernel<<<cdiv(n4, WG), WG, 0, s>>>(n4, x, out);
  return hipGetLastError();
}

hipError_t launch_layernorm(int M, int N, const float* x, int ldx, const float* gamma, const float* beta, float* out, int ldo,
                            hipStream_t s) {
  layernorm_kernel<<<M, WG, 0, s>>>(N, x, ldx, gamma, beta, out, ldo);
  return hipGetLastError();
}

hipError_t launch_transpose(int rows, int cols, const float* in, float* out, hipStream_t s) {
  transpose_kernel<<<dim3((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32)), 256, 0, s>>>(rows, cols, in, out);
  return hipGetLastError();
}

hipError_t launch_softmax(int M, int N, const float* x, float* out, bool transpose, hipStream_t s) {
  if (transpose) softmax_kernel<true><<<M, WG, 0, s>>>(M, N, x, out);
  else softmax_kernel<false><<<M, WG, 0, s>>>(M, N, x, out);
  return hipGetLastError();
}

hipError_t launch_embed(const int32_t* idx, int T, int d, int pos0, const float* wte, const float* wpe, float* out, hipStream_t s) {
  embed_kernel<<<T, WG, 0, s>>>(idx, d, pos0, wte, wpe, out);
  return hipGetLastError();
}

hipError_t launch_vocab_gemv(int V, int d, const float* x, const float* wte, float* logits, hipStream_t s) {
  const int rows_per_wg = NWAVE * VOCAB_ROWS_PER_WAVE;
  vocab_gemv_kernel<<<cdiv(V, rows_per_wg), WG, sizeof(float) * d, s>>>(V, d, x, wte, logits);
  return hipGetLastError();
}

hipError_t launch_attention(int Tq, int pos0, int H, int hs, float scale, const float* q, int ldq, const float* Kc,
                            const float* Vc, size_t hstride, int ldkv, float* out, int ldo, hipStream_t s) {
  // a block of 32 queries per workgroup on the matrix cores
  if (hs == AHS && Tq >= AMQ) {
    static_assert(AHS * AMOST + 2 * AMQ <= AM_WAVE_FLOATS, "merge area must fit a wave's tile area");
    // eight waves once the longest query block has more than eight key tiles
    const bool wide = cdiv(pos0 + Tq, AMK) > 8;
    const size_t lds = sizeof(float) * (wide ? 8 : 4) * AM_WAVE_FLOATS;
    static bool enabled = false;
    if (!enabled) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_mfma_kernel<4>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)(sizeof(float) * 4 * AM_WAVE_FLOATS));
      if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_mfma_kernel<8>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)(sizeof(float) * 8 * AM_WAVE_FLOATS));
      if (e != hipSuccess) return e;
      enabled = true;
    }
    if (wide) attention_mfma_kernel<8><<<dim3(H, cdiv(Tq, AMQ)), 512, lds, s>>>(Tq, pos0, scale, q, ldq, Kc, Vc, hstride, ldkv, out, ldo);
    else attention_mfma_kernel<4><<<dim3(H, cdiv(Tq, AMQ)), 256, lds, s>>>(Tq, pos0, scale, q, ldq, Kc, Vc, hstride, ldkv, out, ldo);
    return hipGetLastError();
  }
  // enough (head, query block) workgroups to fill the GPU; else one workgroup per query row
  if (hs == AHS && Tq >= ATQ && H * cdiv(Tq, ATQ) >= 128) {
    attention_tile_kernel<<<dim3(H, cdiv(Tq, ATQ)), WG, 0, s>>>(Tq, pos0, scale, q, ldq, Kc, Vc, hstride, ldkv, out, ldo);
    return hipGetLastError();
  }
  int lpk = 1;
  while (lpk * 4 < hs) lpk <<= 1;
  if (lpk > 64 || hs > 256 || (hs & 3)) return hipErrorInvalidValue;
  const size_t smem = sizeof(float) * (size_t)(pos0 + Tq);
  if (smem > 48 * 1024) return hipErrorInvalidValue;
  attention_kernel<<<dim3(H, Tq), WG, smem, s>>>(pos0, hs, lpk, scale, q, ldq, Kc, Vc, hstride, ldkv, out, ldo);
  return hipGetLastError();
}

hipError_t launch_copy_rows(int rows, int cols, const float* src, int lds, float* dst, int ldd, hipStream_t s) {
  copy_rows_kernel<<<dim3(cdiv(cols >> 2, WG), rows), WG, 0, s>>>(cols >> 2, src, lds, dst, ldd);
  return hipGetLastError();
}

hipError_t launch_kv_append(int T, int d, int hs, int ctx, int pos0, const float* qkv, float* Kc, float* Vc, hipStream_t s) {
  kv_append_kernel<<<T, WG, 0, s>>>(d, hs, ctx, pos0, qkv, Kc, Vc);
  return hipGetLastError();
}

hipError_t launch_sample_topk(int V, int k, double temperature, const double* u, const float* logits, int32_t* tok,
                              int32_t* out, int slot, int32_t* ids, double* probs, hipStream_t s) {
  if (V < 1 || V > SAMPLE_MAX_V || k < 1 || k > SAMPLE_MAX_K) return hipErrorInvalidValue;
  if (V <= 65536) sample_topk_kernel<true><<<1, 1024, 0, s>>>(V, k, temperature, u, logits, tok, out, slot, ids, probs);
  else sample_topk_kernel<false><<<1, 1024, 0, s>>>(V, k, temperature, u, logits, tok, out, slot, ids, probs);
  return hipGetLastError();
}

hipError_t launch_gemv_slab(int N, int K, const void* slab, bool int8, const float* scale, const float* x, int row_mode,
                            const float* gamma, const float* beta, const float* bias, float* C, int epi, const float* resid,
                            const KvAfter* kv, const int* pos, hipStream_t s, const AttnSlices* merge) {
  if ((K & 3) || N < 1) return hipErrorInvalidValue;
  if (merge && (row_mode != GEMV_ROW_PLAIN || merge->nslice < 1 || merge->nmerge < 1 || merge->nmerge > merge->nslice || merge->hs < 4 ||
                (merge->hs & 3) || K % merge->hs))
    return hipErrorInvalidValue;
  const int S = cdiv(K, 256);
  const size_t lds = sizeof(float) * (size_t)S * 256;
  if (lds > 48 * 1024) return hipErrorInvalidValue;
  GemvSlabArgs a{N, K, S, slab, scale, merge ? merge->part : x, merge ? (int)ROW_MERGE : row_mode, gamma, beta, bias, epi, resid, C,
                 kv ? kv->Kc : nullptr, kv ? kv->Vc : nullptr, kv ? kv->d : 0, kv ? kv->hs : 1, kv ? kv->ctx : 0, pos,
                 merge ? merge->nslice : 0, merge ? merge->hs : 1, merge ? merge->nmerge : 0};
  if (int8) {
    if (N >= 4096) gemv_slab_kernel<4, true><<<cdiv(N, NWAVE * 4), WG, lds, s>>>(a);
    else gemv_slab_kernel<2, true><<<cdiv(N, NWAVE * 2), WG, lds, s>>>(a);
  } else {
    if (N >= 2048) gemv_slab_kernel<2, false><<<cdiv(N, NWAVE * 2), WG, lds, s>>>(a);
    else gemv_slab_kernel<1, false><<<cdiv(N, NWAVE), WG, lds, s>>>(a);
  }
  return hipGetLastError();
}

hipError_t launch_embed_at(const int32_t* tok, int d, const int* pos, const float* wte, const float* wpe, float* x, hipStream_t s) {
  embed_kernel<<<1, WG, 0, s>>>(tok, d, 0, wte, wpe, x, pos);
  return hipGetLastError();
}

hipError_t launch_attention_decode(int H, int hs, int ctx, float scale, const float* q, const float* Kc, const float* Vc, float* out,
                                   const int* pos, hipStream_t s) {
  int lpk = 1;
  while (lpk * 4 < hs) lpk <<= 1;
  if (lpk > 64 || hs > 256 || (hs & 3)) return hipErrorInvalidValue;
  const size_t smem = sizeof(float) * (size_t)ctx;  // scores of the longest context: the launch is the same at every position
  if (smem > 48 * 1024) return hipErrorInvalidValue;
  attention_decode_kernel<<<H, WG, smem, s>>>(hs, lpk, ctx, scale, q, Kc, Vc, (size_t)ctx * hs, out, pos);
  return hipGetLastError();
}

int attention_decode_slice_positions(int hs) {
  int lpk = 1;
  while (lpk * 4 < hs) lpk <<= 1;
  return lpk > 64 ? 0 : ADS_ROWS * (WG / lpk);
}

int attention_decode_slices(int hs, int ctx) {
  const int p = attention_decode_slice_positions(hs);
  return p ? cdiv(ctx, p) : 0;
}

hipError_t launch_attention_decode_slices(int H, int hs, int ctx, float scale, const float* q, const float* Kc, const float* Vc,
                                          const AttnSlices* out, const int* pos, int spec_pos, hipStream_t s) {
  int lpk = 1;
  while (lpk * 4 < hs) lpk <<= 1;
  if (lpk > 64 || hs > 256 || (hs & 3) || !out || out->hs != hs || out->nslice != attention_decode_slices(hs, ctx)) return hipErrorInvalidValue;
  const size_t smem = sizeof(float) * ADS_ROWS * (WG / lpk);
  attention_decode_slice_kernel<<<dim3(H, out->nslice), WG, smem, s>>>(hs, lpk, ctx, scale, q, Kc, Vc, (size_t)ctx * hs, out->part, pos,
                                                                       spec_pos);
  return hipGetLastError();
}

hipError_t launch_vocab_gemv_ln(int V, int d, const float* x, const float* gamma, const float* beta, const float* wte, float* logits,
                                int* pos, hipStream_t s) {
  const int rows_per_wg = NWAVE * VOCAB_ROWS_PER_WAVE;
  vocab_gemv_ln_kernel<<<cdiv(V, rows_per_wg), WG, sizeof(float) * d, s>>>(V, d, x, gamma, beta, wte, logits, pos);
  return hipGetLastError();
}

hipError_t launch_argmax(int V, const float* logits, int32_t* tok, int32_t* out, int slot, hipStream_t s) {
  argmax_kernel<<<1, 1024, 0, s>>>(V, logits, tok, out, slot);
  return hipGetLastError();
}

}  // namespace wgpt
