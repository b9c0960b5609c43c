// Whole-token persistent decode kernel for gfx950.
//
// One launch runs `nsteps` greedy decode steps of GPT.run() (model.js:118-240) at
// batch 1. The reference issues 18 compute passes per layer; a kernel per pass
// cannot reach HBM speed here because one pass moves only 2-9 MB. Instead one
// workgroup per compute unit stays resident for the whole token and the passes
// become phases of a dataflow:
//
//   - every linear layer is split by output columns over the workgroups; a
//     workgroup's share of W is a contiguous slab laid out at load time so that
//     each wave reads 1 KB per instruction (float4 per lane);
//   - the slab of a phase is requested into registers two phases ahead, so HBM
//     streams continuously while the dependent arithmetic of earlier phases runs;
//   - phases exchange their (small) output vectors through global memory as
//     {value, epoch} 64-bit words written and polled with device-scope relaxed
//     atomics: the epoch makes each word self-validating, so no barrier and no
//     ordering between separate stores is needed, and a hop costs one store plus
//     one load round trip;
//   - attention runs on H*SPLIT workgroups (head x slice of the positions) over a
//     head-major KV cache and is merged by every consumer (flash-decoding style);
//   - the vocabulary projection streams wte[V,d] rows (already contiguous in the
//     contraction index), followed by a distributed arg-max that every workgroup
//     finishes redundantly, so the next token needs no broadcast hop.
//
// Every wait is bounded: a poll that does not complete within SPIN_LIMIT rounds
// raises the error word and the workgroup leaves; all others then follow.
#include "decode_persistent.h"

#include <cstdio>

namespace wgpt {

namespace {

typedef unsigned long long u64;

constexpr int NT = PD_THREADS;       // threads per workgroup
constexpr int NW = NT / 64;          // waves per workgroup
constexpr int SEG = 256;             // contraction elements per item (64 lanes x float4)
#ifndef WGPT_NPMAX
#define WGPT_NPMAX 8
#endif
constexpr int NPMAX = WGPT_NPMAX;   // a poll covers up to NPMAX*NT words
constexpr unsigned SPIN_LIMIT = 1u << 18;

__device__ __forceinline__ u64 ld_word(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_word(u64* p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void publish(u64* p, float v, unsigned epoch) { st_word(p, ((u64)epoch << 32) | __float_as_uint(v)); }

// Returns v unchanged but opaque to the optimiser: address arithmetic built on the
// result cannot be hoisted out of the enclosing loops and kept in registers for the
// whole kernel (which otherwise costs more registers than the kernel has).
__device__ __forceinline__ int opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Same for a wave-uniform value held in a scalar register.
__device__ __forceinline__ int opaque_s(int v) {
  asm volatile("" : "+s"(v));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

__device__ __forceinline__ float gelu_ref(float x) {  // instructions.js:718-727
  const float x3 = x * x * x;
  const float cdf = 0.5f * (1.0f + tanhf(0.7978845608f * (x + 0.044715f * x3)));
  float r = x * cdf;
  r = x < -10.0f ? 0.0f : r;
  r = x > 10.0f ? x : r;
  return r;
}

struct Shared {
  int bail;
  float red[2 * NW];
  float red_idx[NW];
};
__shared__ Shared sh;

// Has any thread of this workgroup given up on a bounded wait?
__device__ __forceinline__ int bail_flag() { return __hip_atomic_load(&sh.bail, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }

// Polls n {value, epoch} words until all carry `epoch`, storing the values to dst
// (LDS). Works in chunks of NPMAX*NT words; all loads of a round are issued before
// any is tested. Returns false after SPIN_LIMIT rounds or when another thread or
// workgroup has already given up.
__device__ __forceinline__ bool poll_words(const u64* __restrict__ buf, int n, unsigned epoch, float* dst, int* err) {
  const int t = opaque(threadIdx.x);
  bool ok = true;
  for (int c0 = 0; c0 < n && ok; c0 += NPMAX * NT) {
    const u64* src = buf + c0;
    float* out = dst + c0;
    const int m = n - c0;
    unsigned pending = 0;
#pragma unroll
    for (int i = 0; i < NPMAX; ++i)
      if (t + i * NT < m) pending |= 1u << i;
    unsigned spins = 0;
    while (pending) {
      u64 pk[NPMAX];
#pragma unroll
      for (int i = 0; i < NPMAX; ++i)
        if (pending & (1u << i)) pk[i] = ld_word((src + i * NT) + t);
#pragma unroll
      for (int i = 0; i < NPMAX; ++i)
        if ((pending & (1u << i)) && (unsigned)(pk[i] >> 32) == epoch) {
          out[t + i * NT] = __uint_as_float((unsigned)pk[i]);
          pending &= ~(1u << i);
        }
      if (pending) {
        ++spins;
        if (spins > SPIN_LIMIT || bail_flag() ||
            ((spins & 255u) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
          sh.bail = 1;
          atomicCAS(err, 0, (int)epoch);
          ok = false;
          break;
        }
      }
    }
  }
  return ok;
}

// Registers of one phase's weight slab share: MAXI float4 per lane plus the bias of
// the column this thread will finish.
template <int MAXI>
struct WSet {
  float4 w[MAXI];
  float bias;
};

// Requests the slab share of this wave. Item j (column j / S, segment j % S of this
// workgroup's columns) is 64 consecutive float4; wave v owns items [v*ipw, (v+1)*ipw).
template <int MAXI>
__device__ __forceinline__ void load_items(WSet<MAXI>& ws, const float4* __restrict__ slab, const PhaseGeom& g, int K,
                                           const float* __restrict__ bias, int wg, int wave, int lane) {
  const int col0 = wg * g.cpw;
  int ncols = g.N - col0;
  ncols = ncols > g.cpw ? g.cpw : ncols;
  const int nitems = ncols > 0 ? ncols * g.S : 0;
  const int ln = opaque(lane);
  const float4* base = slab + (size_t)wg * g.cpw * g.S * 64;
  int j = opaque_s(wave) * g.ipw;
  int seg = j % g.S;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (i < g.ipw && j < nitems && seg * SEG + ln * 4 < K) v = (base + (size_t)j * 64)[ln];
    ws.w[i] = v;
    ++j;
    if (++seg == g.S) seg = 0;
  }
  ws.bias = ((int)threadIdx.x < ncols) ? bias[col0 + threadIdx.x] : 0.f;
}

// Dot products of this wave's items with the input vector xs (LDS, zero padded up
// to S*SEG). Per (column, wave) partial sums go to part[col*NW + wave].
template <int MAXI>
__device__ __forceinline__ void gemv_items(const WSet<MAXI>& ws, const float* xs, float* part, const PhaseGeom& g, int wg,
                                           int wave, int lane) {
  const int col0 = wg * g.cpw;
  int ncols = g.N - col0;
  ncols = ncols > g.cpw ? g.cpw : ncols;
  const int nitems = ncols > 0 ? ncols * g.S : 0;
  int j = opaque_s(wave) * g.ipw;
  int col = j / g.S;
  int seg = j - col * g.S;
  float acc = 0.f;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    if (i < g.ipw && j < nitems) {
      const float4 x = *reinterpret_cast<const float4*>(xs + seg * SEG + lane * 4);
      const float4 w = ws.w[i];
      acc += (w.x * x.x + w.y * x.y) + (w.z * x.z + w.w * x.w);
      if (seg == g.S - 1 || i == g.ipw - 1 || j == nitems - 1) {
        const float r = wave_sum(acc);
        if (lane == 0) part[col * NW + wave] = r;
        acc = 0.f;
      }
      ++j;
      if (++seg == g.S) {
        seg = 0;
        ++col;
      }
    }
  }
}

// Sum of the per-wave partials of local column c, in ascending wave order.
__device__ __forceinline__ float column_sum(const float* part, const PhaseGeom& g, int c) {
  c = opaque(c);
  const int v0 = (c * g.S) / g.ipw;
  int v1 = ((c + 1) * g.S - 1) / g.ipw;
  v1 = v1 > NW - 1 ? NW - 1 : v1;
  float s = 0.f;
  for (int v = v0; v <= v1; ++v) s += part[c * NW + v];
  return s;
}

// LayerNorm of xs[0..d) in place (instructions.js:451-550 semantics: biased
// variance about the mean, eps inside the sqrt, true division).
__device__ __forceinline__ void layernorm_lds(float* xs, int d, const float* __restrict__ gamma,
                                              const float* __restrict__ beta) {
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  float s = 0.f;
  for (int e = threadIdx.x; e < d; e += NT) s += xs[e];
  s = wave_sum(s);
  if (lane == 0) sh.red[wave] = s;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int v = 0; v < NW; ++v) tot += sh.red[v];
  const float mean = tot / (float)d;
  float q = 0.f;
  for (int e = threadIdx.x; e < d; e += NT) {
    const float a = xs[e] - mean;
    q += a * a;
  }
  q = wave_sum(q);
  if (lane == 0) sh.red[NW + wave] = q;
  __syncthreads();
  float var = 0.f;
#pragma unroll
  for (int v = 0; v < NW; ++v) var += sh.red[NW + v];
  const float stdev = sqrtf(var / (float)d + 1e-5f);
  for (int e = threadIdx.x; e < d; e += NT) xs[e] = gamma[e] * ((xs[e] - mean) / stdev) + beta[e];
  __syncthreads();
}

template <int MAXI, int MAXKV>
__global__ __launch_bounds__(NT) void decode_persistent_kernel(PersistentArgs a) {
  extern __shared__ float lds[];

  // LDS carve-up (floats): xs [a.xs_floats] | att partials [a.attp_floats] | part | qkv_s | own residual
  float* xs = lds;
  float* attp = xs + a.xs_floats;
  float* part = attp + a.attp_floats;
  float* qkv_s = part + a.part_floats;

  const int wg = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: same for the whole wave
  const int d = a.d, hs = a.hs, H = a.H, hid = 4 * a.d;
  if (tid == 0) sh.bail = 0;
  for (int e = tid; e < a.xs_floats; e += NT) xs[e] = 0.f;
  __syncthreads();

  // attention role: head and slice of the positions
  const bool att_role = wg < H * a.split;
  const int ah = wg / a.split, as = wg - ah * a.split;
  // attention threads: 32 key groups (tid >> 4) of 16 lanes (tid & 15), hs = 64

  // columns this workgroup finishes in the d-wide phases (C and E share geometry N = d)
  const int colC0 = wg * a.gC.cpw;
  int ncolC = d - colC0;
  ncolC = ncolC > a.gC.cpw ? a.gC.cpw : (ncolC < 0 ? 0 : ncolC);

  WSet<MAXI> set0, set1;
  unsigned ep = a.ebase;
  int tok = a.tok[0];

  const LayerParamOffsets po = layer_param_offsets(d);
  load_items<MAXI>(set0, a.slabs, a.gA, d, a.lparams + po.bA, wg, wave, lane);

  for (int step = 0; step < a.nsteps; ++step) {
    const int pos = a.pos0 + step;
    // ---- embedding: every workgroup builds the row itself (instructions.js:795-821) ----
    for (int e = tid; e < d; e += NT) xs[e] = a.wte[(size_t)tok * d + e] + a.wpe[(size_t)pos * d + e];
    __syncthreads();

    // slice of positions 0..pos for the attention role
    const int nkeys = pos + 1;
    const int chunk = (nkeys + a.split - 1) / a.split;
    const int c0 = as * chunk;
    int c1 = c0 + chunk;
    c1 = c1 > nkeys ? nkeys : c1;

    for (int li = 0; li < a.L; ++li) {
      const float4* slab = a.slabs + (size_t)li * a.slab_stride;
      const float* lp = a.lparams + (size_t)li * po.stride;
      float* Kc = a.kv + ((size_t)(li * 2 + 0) * H + ah) * a.ctx * hs;
      float* Vc = a.kv + ((size_t)(li * 2 + 1) * H + ah) * a.ctx * hs;

      // ================= phase A: LN1 + QKV =================
      if (li > 0) {
        if (!poll_words(a.bufR2, d, ep, xs, a.err)) {}
        __syncthreads();
        if (sh.bail) return;
      }
      const float own_r = tid < ncolC ? xs[colC0 + tid] : 0.f;  // residual of the columns finished in phase C
      layernorm_lds(xs, d, lp + po.ln1g, lp + po.ln1b);
      // request what is needed two phases ahead: proj weights and this layer's cached keys/values
      load_items<MAXI>(set1, slab + a.slab_offC, a.gC, d, lp + po.bC, wg, wave, lane);
      float4 kreg[MAXKV], vreg[MAXKV];
      if (att_role) {
        const int g16 = opaque(tid >> 4), sub = opaque(tid & 15);
#pragma unroll
        for (int i = 0; i < MAXKV; ++i) {
          const int j = c0 + g16 + 32 * i;
          float4 kk = make_float4(0.f, 0.f, 0.f, 0.f), vv = kk;
          if (j < c1 && j < pos) {
            const u64* kp = reinterpret_cast<const u64*>(Kc + (size_t)j * hs + sub * 4);
            const u64* vp = reinterpret_cast<const u64*>(Vc + (size_t)j * hs + sub * 4);
            const u64 k0 = ld_word(kp), k1 = ld_word(kp + 1), v0 = ld_word(vp), v1 = ld_word(vp + 1);
            kk = make_float4(__uint_as_float((unsigned)k0), __uint_as_float((unsigned)(k0 >> 32)),
                             __uint_as_float((unsigned)k1), __uint_as_float((unsigned)(k1 >> 32)));
            vv = make_float4(__uint_as_float((unsigned)v0), __uint_as_float((unsigned)(v0 >> 32)),
                             __uint_as_float((unsigned)v1), __uint_as_float((unsigned)(v1 >> 32)));
          }
          kreg[i] = kk;
          vreg[i] = vv;
        }
      }
      gemv_items<MAXI>(set0, xs, part, a.gA, wg, wave, lane);
      __syncthreads();
      ++ep;
      {
        const int col0 = wg * a.gA.cpw;
        int ncols = 3 * d - col0;
        ncols = ncols > a.gA.cpw ? a.gA.cpw : ncols;
        if (tid < ncols) publish(a.bufQKV + col0 + tid, column_sum(part, a.gA, tid) + set0.bias, ep);
      }

      // ================= phase B: attention slice =================
      // fc weights go where the QKV weights were
      load_items<MAXI>(set0, slab + a.slab_offD, a.gD, d, lp + po.bD, wg, wave, lane);
      ++ep;
      if (att_role) {
        // q, k, v of this head for the new token
        {
          unsigned pending = tid < 3 * hs ? 1u : 0u;
          unsigned spins = 0;
          const int which = tid / hs, e = tid - which * hs;
          const u64* src = a.bufQKV + which * d + ah * hs + e;
          while (pending) {
            const u64 pk = ld_word(src);
            if ((unsigned)(pk >> 32) == ep - 1) {
              qkv_s[tid] = __uint_as_float((unsigned)pk);
              pending = 0;
            } else if (++spins > SPIN_LIMIT || bail_flag()) {
              sh.bail = 1;
              atomicCAS(a.err, 0, (int)ep);
              break;
            }
          }
        }
        __syncthreads();
        if (sh.bail) return;
        // the slice that holds the new position appends it to the cache and uses it from LDS
        const bool has_new = pos >= c0 && pos < c1;
        if (has_new && tid < 32) {
          const float* src = qkv_s + (tid < 16 ? hs : 2 * hs) + (tid & 15) * 4;
          float* dstp = (tid < 16 ? Kc : Vc) + (size_t)pos * hs + (tid & 15) * 4;
          u64* dp = reinterpret_cast<u64*>(dstp);
          st_word(dp, ((u64)__float_as_uint(src[1]) << 32) | __float_as_uint(src[0]));
          st_word(dp + 1, ((u64)__float_as_uint(src[3]) << 32) | __float_as_uint(src[2]));
        }
        const int g16 = opaque(tid >> 4), sub = opaque(tid & 15);
        const float4 qv = *reinterpret_cast<const float4*>(qkv_s + sub * 4);
        float sc[MAXKV];
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < MAXKV; ++i) {
          const int j = c0 + g16 + 32 * i;
          if (j == pos && has_new) {
            kreg[i] = *reinterpret_cast<const float4*>(qkv_s + hs + sub * 4);
            vreg[i] = *reinterpret_cast<const float4*>(qkv_s + 2 * hs + sub * 4);
          }
          float p = (qv.x * kreg[i].x + qv.y * kreg[i].y) + (qv.z * kreg[i].z + qv.w * kreg[i].w);
          p += __shfl_xor(p, 8);
          p += __shfl_xor(p, 4);
          p += __shfl_xor(p, 2);
          p += __shfl_xor(p, 1);
          sc[i] = j < c1 ? p * a.scale : -INFINITY;
          m = fmaxf(m, sc[i]);
        }
        m = fmaxf(m, __shfl_xor(m, 16));
        m = fmaxf(m, __shfl_xor(m, 32));
        if (lane == 0) sh.red[wave] = m;
        __syncthreads();
#pragma unroll
        for (int v = 0; v < NW; ++v) m = fmaxf(m, sh.red[v]);
        float l = 0.f;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
        if (m > -INFINITY) {
#pragma unroll
          for (int i = 0; i < MAXKV; ++i) {
            const float p = sc[i] > -INFINITY ? expf(sc[i] - m) : 0.f;
            l += p;
            o.x += p * vreg[i].x; o.y += p * vreg[i].y; o.z += p * vreg[i].z; o.w += p * vreg[i].w;
          }
        }
        // combine the 32 key groups: 4 per wave by shuffles, then 8 waves through LDS
        o.x += __shfl_xor(o.x, 16); o.y += __shfl_xor(o.y, 16); o.z += __shfl_xor(o.z, 16); o.w += __shfl_xor(o.w, 16);
        o.x += __shfl_xor(o.x, 32); o.y += __shfl_xor(o.y, 32); o.z += __shfl_xor(o.z, 32); o.w += __shfl_xor(o.w, 32);
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        __syncthreads();  // sh.red reads above are done
        if (lane < 16) *reinterpret_cast<float4*>(part + wave * (hs + 4) + lane * 4) = o;
        if (lane == 0) part[wave * (hs + 4) + hs] = l;
        __syncthreads();
        if (tid < hs + 2) {
          float v = 0.f;
          if (tid < hs) {
#pragma unroll
            for (int w8 = 0; w8 < NW; ++w8) v += part[w8 * (hs + 4) + tid];
          } else if (tid == hs) {
            v = m;
          } else {
#pragma unroll
            for (int w8 = 0; w8 < NW; ++w8) v += part[w8 * (hs + 4) + hs];
          }
          publish(a.bufATT + (size_t)wg * (hs + 2) + tid, v, ep);
        }
      }

      // ================= phase C: merge slices, projection, residual =================
      if (!poll_words(a.bufATT, H * a.split * (hs + 2), ep, attp, a.err)) {}
      __syncthreads();
      if (sh.bail) return;
      for (int e = tid; e < d; e += NT) {
        const int h = e / hs, c = e - h * hs;
        const float* ph = attp + (size_t)h * a.split * (hs + 2);
        float M = -INFINITY;
        for (int s2 = 0; s2 < a.split; ++s2) M = fmaxf(M, ph[s2 * (hs + 2) + hs]);
        float Lsum = 0.f, val = 0.f;
        for (int s2 = 0; s2 < a.split; ++s2) {
          const float ms = ph[s2 * (hs + 2) + hs];
          const float wgt = ms > -INFINITY ? expf(ms - M) : 0.f;
          Lsum += ph[s2 * (hs + 2) + hs + 1] * wgt;
          val += ph[s2 * (hs + 2) + c] * wgt;
        }
        xs[e] = val / Lsum;
      }
      __syncthreads();
      // fc2 weights go where the projection weights are, after they have been used:
      gemv_items<MAXI>(set1, xs, part, a.gC, wg, wave, lane);
      __syncthreads();
      ++ep;
      float r1 = 0.f;
      if (tid < ncolC) {
        r1 = column_sum(part, a.gC, tid) + set1.bias + own_r;
        publish(a.bufR1 + colC0 + tid, r1, ep);
      }
      load_items<MAXI>(set1, slab + a.slab_offE, a.gE, hid, lp + po.bE, wg, wave, lane);

      // ================= phase D: LN2 + fc + GELU =================
      if (!poll_words(a.bufR1, d, ep, xs, a.err)) {}
      __syncthreads();
      if (sh.bail) return;
      layernorm_lds(xs, d, lp + po.ln2g, lp + po.ln2b);
      gemv_items<MAXI>(set0, xs, part, a.gD, wg, wave, lane);
      __syncthreads();
      ++ep;
      {
        const int col0 = wg * a.gD.cpw;
        int ncols = hid - col0;
        ncols = ncols > a.gD.cpw ? a.gD.cpw : ncols;
        if (tid < ncols) publish(a.bufH + col0 + tid, gelu_ref(column_sum(part, a.gD, tid) + set0.bias), ep);
      }
      // next layer's QKV weights (or nothing after the last layer)
      if (li + 1 < a.L) load_items<MAXI>(set0, slab + a.slab_stride, a.gA, d, lp + po.stride + po.bA, wg, wave, lane);
      else if (step + 1 < a.nsteps) load_items<MAXI>(set0, a.slabs, a.gA, d, a.lparams + po.bA, wg, wave, lane);

      // ================= phase E: fc2 + residual =================
      if (!poll_words(a.bufH, hid, ep, xs, a.err)) {}
      __syncthreads();
      if (sh.bail) return;
      gemv_items<MAXI>(set1, xs, part, a.gE, wg, wave, lane);
      __syncthreads();
      ++ep;
      if (tid < ncolC) publish(a.bufR2 + colC0 + tid, column_sum(part, a.gE, tid) + set1.bias + r1, ep);
      // xs beyond d must be zero again for the d-wide phases that follow
      for (int e = d + tid; e < a.xs_floats; e += NT) xs[e] = 0.f;
      __syncthreads();
    }

    // ================= final LayerNorm + vocabulary projection =================
    if (!poll_words(a.bufR2, d, ep, xs, a.err)) {}
    __syncthreads();
    if (sh.bail) return;
    layernorm_lds(xs, d, a.lnf_g, a.lnf_b);
    {
      const int v0 = wg * a.rows_per_wg;
      int v1 = v0 + a.rows_per_wg;
      v1 = v1 > a.V ? a.V : v1;
      float best = -INFINITY;
      int besti = 0x7fffffff;
      const int S = a.gA.S;
      for (int vb = v0 + wave * 4; vb < v1; vb += NW * 4) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int s2 = 0; s2 < S; ++s2) {
          const int k = s2 * SEG + lane * 4;
          if (k < d) {
            const float4 x = *reinterpret_cast<const float4*>(xs + k);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              if (vb + r < v1) {
                const float4 w = *reinterpret_cast<const float4*>(a.wte + (size_t)(vb + r) * d + k);
                acc[r] += (w.x * x.x + w.y * x.y) + (w.z * x.z + w.w * x.w);
              }
            }
          }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float s = wave_sum(acc[r]);
          if (vb + r < v1) {
            if (lane == 0) a.logits[vb + r] = s;
            if (s > best || besti == 0x7fffffff) {
              best = s;
              besti = vb + r;
            }
          }
        }
      }
      if (lane == 0) {
        sh.red[wave] = best;
        sh.red_idx[wave] = __int_as_float(besti);
      }
      __syncthreads();
      ++ep;
      if (tid == 0) {
        float b = sh.red[0];
        int bi = __float_as_int(sh.red_idx[0]);
        for (int v = 1; v < NW; ++v) {
          const float ov = sh.red[v];
          const int oi = __float_as_int(sh.red_idx[v]);
          if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > b || (ov == b && oi < bi))) {
            b = ov;
            bi = oi;
          }
        }
        publish(a.bufAM + 2 * wg, b, ep);
        publish(a.bufAM + 2 * wg + 1, __int_as_float(bi), ep);
      }
    }
    // ================= arg-max over the workgroups, finished by everyone =================
    if (!poll_words(a.bufAM, 2 * a.G, ep, attp, a.err)) {}
    __syncthreads();
    if (sh.bail) return;
    {
      float b = -INFINITY;
      int bi = 0x7fffffff;
      for (int w2 = lane; w2 < a.G; w2 += 64) {
        const float ov = attp[2 * w2];
        const int oi = __float_as_int(attp[2 * w2 + 1]);
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > b || (ov == b && oi < bi))) {
          b = ov;
          bi = oi;
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(b, off);
        const int oi = __shfl_xor(bi, off);
        if (oi != 0x7fffffff && (bi == 0x7fffffff || ov > b || (ov == b && oi < bi))) {
          b = ov;
          bi = oi;
        }
      }
      tok = bi;  // every wave of every workgroup holds the same result
      if (wg == 0 && tid == 0) a.out_tok[step] = tok;
    }
    __syncthreads();
  }
}

__global__ void build_slab_kernel(const float* __restrict__ W, int ldw, int K, int N, int cpw, int S, size_t total,
                                  float4* __restrict__ slab) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  const size_t it = idx >> 6;
  const int per_wg = cpw * S;
  const int w = (int)(it / per_wg), j = (int)(it - (size_t)w * per_wg);
  const int c = j / S, seg = j - c * S;
  const int col = w * cpw + c, k = seg * SEG + lane * 4;
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (col < N)
    for (int e = 0; e < 4; ++e)
      if (k + e < K) v[e] = W[(size_t)(k + e) * ldw + col];
  slab[idx] = make_float4(v[0], v[1], v[2], v[3]);
}

template <int MAXI, int MAXKV>
hipError_t launch_t(const PersistentArgs& a, size_t lds_bytes, hipStream_t s) {
  auto kern = decode_persistent_kernel<MAXI, MAXKV>;
  static size_t allowed = 0;  // dynamic LDS size already enabled for this instantiation
  if (lds_bytes > allowed) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    allowed = lds_bytes;
  }
  kern<<<a.G, NT, lds_bytes, s>>>(a);
  return hipGetLastError();
}

}  // namespace

PhaseGeom make_geom(int N, int K, int G) {
  PhaseGeom g;
  g.N = N;
  g.cpw = (N + G - 1) / G;
  g.S = (K + SEG - 1) / SEG;
  g.ipw = (g.cpw * g.S + NW - 1) / NW;
  return g;
}

size_t slab_float4s(const PhaseGeom& g, int G) { return (size_t)G * g.cpw * g.S * 64; }

hipError_t build_slab(const float* W, int ldw, int K, const PhaseGeom& g, int G, float4* slab, hipStream_t s) {
  const size_t total = slab_float4s(g, G);
  build_slab_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(W, ldw, K, g.N, g.cpw, g.S, total, slab);
  return hipGetLastError();
}

int persistent_max_items(const PersistentArgs& a) {
  int m = a.gA.ipw;
  m = a.gC.ipw > m ? a.gC.ipw : m;
  m = a.gD.ipw > m ? a.gD.ipw : m;
  m = a.gE.ipw > m ? a.gE.ipw : m;
  return m;
}

size_t persistent_lds_bytes(const PersistentArgs& a) {
  const size_t need = sizeof(float) * ((size_t)a.xs_floats + a.attp_floats + a.part_floats + 3 * a.hs + 16);
  // more than half of a compute unit's 160 KB, so that exactly one workgroup lives on each
  const size_t one_per_cu = 84 * 1024;
  return need > one_per_cu ? need : one_per_cu;
}

hipError_t launch_decode_persistent(const PersistentArgs& a, hipStream_t s) {
  const int mi = persistent_max_items(a);
  const size_t lds = persistent_lds_bytes(a);
  const int kv_per_thread = ((a.ctx + a.split - 1) / a.split + 31) / 32;
  if (kv_per_thread > 8) return hipErrorInvalidValue;
  if (mi <= 4) return launch_t<4, 8>(a, lds, s);
  if (mi <= 8) return launch_t<8, 8>(a, lds, s);
  if (mi <= 16) return launch_t<16, 8>(a, lds, s);
  return hipErrorInvalidValue;
}

}  // namespace wgpt
