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
//   - the slab of a phase is requested into registers a phase ahead (right after the
//     poll that starts the phase before it, where two register sets fit), so it
//     lands while that phase computes and never queues in front of a poll;
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
// Every wait is bounded: a poll that does not complete within `spin_limit` rounds
// raises the error word; every later wait of every workgroup then ends at once and
// the launch drains.
#include "decode_persistent.h"

#include <cstdio>
#include <type_traits>

namespace wgpt {

namespace {

typedef unsigned long long u64;

constexpr int NT = PD_THREADS;       // threads per workgroup
constexpr int NW = NT / 64;          // waves per workgroup
constexpr int SEG = 256;             // contraction elements per item (64 lanes x float4)

__device__ __forceinline__ u64 ld_word(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_word(u64* p, u64 v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void publish(u64* p, float v, unsigned epoch) { st_word(p, ((u64)epoch << 32) | __float_as_uint(v)); }

// Three values and one epoch in 16 bytes, written by one 128-bit store of one lane and polled by one 128-bit load
// (poll_triples): a naturally aligned 16-byte access of a lane is one transaction on both sides, so the epoch
// validates the three values it travels with. What a hop costs beyond its latency goes with the number of poll
// instructions, and a consumer reads a third fewer of these than of {value, epoch} pairs.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void publish3(u64* p, float v0, float v1, float v2, unsigned epoch) {
  u32x4 pk;
  pk.x = __float_as_uint(v0);
  pk.y = __float_as_uint(v1);
  pk.z = __float_as_uint(v2);
  pk.w = epoch;
  asm volatile("global_store_dwordx4 %0, %1, off sc1" : : "v"(p), "v"(pk) : "memory");
}

// Streaming (non-temporal) 128-bit load: weights are read once per token and must
// not displace the small hot data (parameters, instructions) from the caches.
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 ld_stream(const float4* p) {
  const f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
  return make_float4(t.x, t.y, t.z, t.w);
}

// Returns v unchanged but opaque to the optimiser: address arithmetic built on the
// result cannot be hoisted out of the enclosing loops and kept in registers for the
// whole kernel (which otherwise costs more registers than the kernel has).
__device__ __forceinline__ int opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}
// One data-parallel-primitive step: v (+|max) the value of another lane selected by
// CTRL, only in the rows of ROWS; lanes without a source contribute the identity.
template <int CTRL, int ROWS>
__device__ __forceinline__ float dpp_add(float v) {
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROWS, 0xf, true));
}
template <int CTRL, int ROWS>
__device__ __forceinline__ float dpp_max(float v) {
  const int ninf = __float_as_int(-INFINITY);
  return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(ninf, __float_as_int(v), CTRL, ROWS, 0xf, false)));
}

// Sum over the 64 lanes, returned as a wave-uniform value. Row-wise inclusive scan
// (row_shr 1,2,4,8), then lane 15 of each row into the next row (row_bcast15) and
// lane 31 into the upper half (row_bcast31): lane 63 holds the total.
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0x111, 0xf>(v);
  v = dpp_add<0x112, 0xf>(v);
  v = dpp_add<0x114, 0xf>(v);
  v = dpp_add<0x118, 0xf>(v);
  v = dpp_add<0x142, 0xa>(v);
  v = dpp_add<0x143, 0xc>(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}
// N sums side by side, step by step: a step's N instructions are independent, so none waits for the one
// before it (one sum after the other is six dependent steps each).
template <int N>
__device__ __forceinline__ void wave_sum_n(float (&v)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = dpp_add<0x111, 0xf>(v[i]);
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = dpp_add<0x112, 0xf>(v[i]);
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = dpp_add<0x114, 0xf>(v[i]);
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = dpp_add<0x118, 0xf>(v[i]);
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = dpp_add<0x142, 0xa>(v[i]);
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = dpp_add<0x143, 0xc>(v[i]);
#pragma unroll
  for (int i = 0; i < N; ++i) v[i] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v[i]), 63));
}
// Maximum / sum over each group of 8 adjacent lanes, every lane of the group gets it: lane ^ 1 and lane ^ 2 inside
// the quad, then the mirrored lane of the half row, which lies in the group's other quad.
template <int CTRL>
__device__ __forceinline__ float dpp_get(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
__device__ __forceinline__ float group8_max(float v) {
  v = fmaxf(v, dpp_get<0xB1>(v));
  v = fmaxf(v, dpp_get<0x4E>(v));
  return fmaxf(v, dpp_get<0x141>(v));
}
__device__ __forceinline__ float group8_sum(float v) {
  v += dpp_get<0xB1>(v);
  v += dpp_get<0x4E>(v);
  return v + dpp_get<0x141>(v);
}
// Sum over each row of 16 lanes, every lane of the row gets it (row rotations).
__device__ __forceinline__ float row16_sum(float v) {
  v = dpp_add<0x128, 0xf>(v);
  v = dpp_add<0x124, 0xf>(v);
  v = dpp_add<0x122, 0xf>(v);
  v = dpp_add<0x121, 0xf>(v);
  return v;
}

// v of lane l and of lane l ^ 16 (l ^ 32) as a pair, through the row (half-wave) swap instructions: plain
// vector instructions, where a shuffle goes through the LDS pipeline.
__device__ __forceinline__ void pair16(float v, float& a, float& b) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void pair32(float v, float& a, float& b) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor16_sum(float v) { float a, b; pair16(v, a, b); return a + b; }
__device__ __forceinline__ float xor32_sum(float v) { float a, b; pair32(v, a, b); return a + b; }
__device__ __forceinline__ float xor16_max(float v) { float a, b; pair16(v, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float xor32_max(float v) { float a, b; pair32(v, a, b); return fmaxf(a, b); }

// Hardware approximations (about 1 ulp each), used where an exact quotient, square
// root or exponential would put a dozen dependent instructions on a phase's
// critical path; the difference is orders of magnitude inside the parity tolerance.
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }

__device__ __forceinline__ float gelu_ref(float x) {  // instructions.js:718-727
  const float x3 = x * x * x;
  // 1 + tanh(u) = 2 - 2 / (1 + exp(2u)); exp overflowing to +inf gives exactly 2, underflowing to 0 gives 0
  const float u = 0.7978845608f * (x + 0.044715f * x3);
  const float cdf = 1.0f - fast_rcp(1.0f + fast_exp(2.0f * u));
  float r = x * cdf;
  r = x < -10.0f ? 0.0f : r;
  r = x > 10.0f ? x : r;
  return r;
}

struct Shared {
  int bail;
  float red[32];
  float red_idx[NW];
  float cand_v[NW * PD_TOPK];  // per-wave top-k candidates of the vocabulary phase
  int cand_i[NW * PD_TOPK];
};
__shared__ Shared sh;

// Has any thread of this workgroup given up on a bounded wait?
__device__ __forceinline__ int bail_flag() { return __hip_atomic_load(&sh.bail, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP); }

// All vector-memory loads issued so far have completed (vmcnt = 0); the other
// counters are left alone. Placed after each poll so that registers requested
// before the poll are known to have landed on every control path.
__device__ __forceinline__ void wait_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// Compile-time geometry of one model shape: everything the phases index with is a
// constant, so the per-phase code is loads, FMAs and a few scalar compares. (A wave
// retires only one instruction every few cycles; index arithmetic on the critical
// path of a phase costs as much as the hop between phases.)
template <int D_, int H_, bool I8_ = false, int SPLIT_ = PD_SPLIT>
struct Shape {
  static constexpr int D = D_, H = H_, HS = D_ / H_, HID = 4 * D_;
  static constexpr bool I8 = I8_;  // linear weights are int8 (4 contraction elements per 32-bit word) + per-column scale
  static constexpr int G = PD_GRID, SPLIT = SPLIT_;  // SPLIT: position slices per head in the attention phase
  static_assert(H * SPLIT <= PD_GRID, "a workgroup per head and slice");
  static constexpr int SD = (D + SEG - 1) / SEG;      // segments of a D-long contraction
  static constexpr int SH = (HID + SEG - 1) / SEG;    // segments of a HID-long contraction
  static constexpr int ATTW = H * SPLIT * (HS + 2);   // values of the attention exchange (three to a word)
  static_assert((HS + 2) % 3 == 0, "a slice's values fill whole words of three");
  static_assert(HS == 64, "the attention phase is laid out for head size 64");
};

// One linear phase: N outputs from a K-long input.
// WHOLE: local column c of a workgroup lives in wave c % NW (as its (c / NW)-th),
// which holds all S items of the column and finishes it (scale, bias, activation) in
// lane c / NW; the finished values meet in LDS so that one wave publishes them with
// one store instruction (a store per wave makes the hop measurably slower).
// Otherwise (the long contraction of the second MLP matrix) the workgroup's items
// are dealt to the waves in runs of IPW, a column is the sum of the partials of
// several waves and thread c finishes column c.
template <int N_, int K_, bool WHOLE_>
struct Phase {
  static constexpr int N = N_, K = K_;
  static constexpr bool WHOLE = WHOLE_;
  static constexpr int CPW = (N + PD_GRID - 1) / PD_GRID;  // columns per workgroup
  static constexpr int S = (K + SEG - 1) / SEG;            // segments (items) per column
  static constexpr int ITEMS = CPW * S;                    // items per workgroup
  static constexpr int CW = (CPW + NW - 1) / NW;           // columns finished per wave
  static constexpr int IPW = WHOLE ? CW * S : (ITEMS + NW - 1) / NW;  // items per wave
  static constexpr bool RAGGED = CPW * PD_GRID != N;       // some workgroups finish fewer than CPW columns
};

// Idles the wave for about 64 * units clocks.
__device__ __forceinline__ void nap(int units) {
  for (int i = 0; i < units; ++i) __builtin_amdgcn_s_sleep(1);
}

// f(std::integral_constant<int, i>) for i = 0 .. N-1.
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) {
  (f(std::integral_constant<int, Is>()), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(f, std::make_integer_sequence<int, N>());
}

// NL 128-bit agent-scope loads (two {value, epoch} words each) issued back to back and waited for together, as ONE
// statement: the compiler does not track loads made in inline assembly, so none of the destinations may be touched
// before the wait that ends the statement. (vmcnt(0) also covers the weight requests in flight: they were issued
// earlier and return first anyway.)
template <int NL>
struct WideLoads;
#define WGPT_WL "global_load_dwordx4 "
#define WGPT_WE ", off sc1\n\t"
template <>
struct WideLoads<1> {
  static __device__ __forceinline__ void run(u32x4 (&v)[1], const u64* const (&p)[1]) {
    asm volatile(WGPT_WL "%0, %1" WGPT_WE "s_waitcnt vmcnt(0)" : "=&v"(v[0]) : "v"(p[0]) : "memory");
  }
};
template <>
struct WideLoads<2> {
  static __device__ __forceinline__ void run(u32x4 (&v)[2], const u64* const (&p)[2]) {
    asm volatile(WGPT_WL "%0, %2" WGPT_WE WGPT_WL "%1, %3" WGPT_WE "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]) : "v"(p[0]), "v"(p[1]) : "memory");
  }
};
template <>
struct WideLoads<3> {
  static __device__ __forceinline__ void run(u32x4 (&v)[3], const u64* const (&p)[3]) {
    asm volatile(WGPT_WL "%0, %3" WGPT_WE WGPT_WL "%1, %4" WGPT_WE WGPT_WL "%2, %5" WGPT_WE "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]) : "v"(p[0]), "v"(p[1]), "v"(p[2]) : "memory");
  }
};
template <>
struct WideLoads<4> {
  static __device__ __forceinline__ void run(u32x4 (&v)[4], const u64* const (&p)[4]) {
    asm volatile(WGPT_WL "%0, %4" WGPT_WE WGPT_WL "%1, %5" WGPT_WE WGPT_WL "%2, %6" WGPT_WE WGPT_WL "%3, %7" WGPT_WE "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]) : "memory");
  }
};
template <>
struct WideLoads<5> {
  static __device__ __forceinline__ void run(u32x4 (&v)[5], const u64* const (&p)[5]) {
    asm volatile(WGPT_WL "%0, %5" WGPT_WE WGPT_WL "%1, %6" WGPT_WE WGPT_WL "%2, %7" WGPT_WE WGPT_WL "%3, %8" WGPT_WE WGPT_WL "%4, %9" WGPT_WE
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4])
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]) : "memory");
  }
};
template <>
struct WideLoads<6> {
  static __device__ __forceinline__ void run(u32x4 (&v)[6], const u64* const (&p)[6]) {
    asm volatile(WGPT_WL "%0, %6" WGPT_WE WGPT_WL "%1, %7" WGPT_WE WGPT_WL "%2, %8" WGPT_WE WGPT_WL "%3, %9" WGPT_WE WGPT_WL "%4, %10" WGPT_WE
                 WGPT_WL "%5, %11" WGPT_WE "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5])
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]) : "memory");
  }
};
template <>
struct WideLoads<7> {
  static __device__ __forceinline__ void run(u32x4 (&v)[7], const u64* const (&p)[7]) {
    asm volatile(WGPT_WL "%0, %7" WGPT_WE WGPT_WL "%1, %8" WGPT_WE WGPT_WL "%2, %9" WGPT_WE WGPT_WL "%3, %10" WGPT_WE WGPT_WL "%4, %11" WGPT_WE
                 WGPT_WL "%5, %12" WGPT_WE WGPT_WL "%6, %13" WGPT_WE "s_waitcnt vmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6])
                 : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]) : "memory");
  }
};
#undef WGPT_WL
#undef WGPT_WE

// Waits for the N words of an exchange (all of epoch `epoch`) and leaves their values in dst[0, N). A thread polls
// PAIRS of adjacent words with one 128-bit load: what a hop costs beyond its latency goes with the number of load
// instructions, not with the bytes (measured with the exchange alone, 256 workgroups: 3072 words 2.01 us with 64-bit
// polls, 1.56 us with 128-bit ones; 6144 words 2.99 and 2.01 us). Each word validates itself, so it does not matter
// whether the two halves of a load are from the same moment; a naturally aligned 8-byte half is never torn.
template <int N>
__device__ __forceinline__ void poll_words(const u64* __restrict__ buf, unsigned epoch, float* dst, int* err, int delay,
                                           unsigned spin_limit) {
  static_assert(N % 2 == 0, "words are polled in pairs");
  constexpr int NPAIR = N / 2;
  constexpr int NP = (NPAIR + NT - 1) / NT;
  constexpr int CH = 7;  // loads per statement; more pairs per thread are fetched in several rounds
  const int t = opaque(threadIdx.x);
  unsigned pending = 0;
  const u64* src[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const bool mine = i * NT + NT <= NPAIR || t + i * NT < NPAIR;
    if (mine) pending |= 1u << i;
    src[i] = buf + 2 * (mine ? t + i * NT : NPAIR - 1);  // (a thread without a pair re-reads the last one)
  }
  unsigned spins = 0;
  nap(delay);
  while (pending) {
    static_for<(NP + CH - 1) / CH>([&](auto CI) {
      constexpr int c0 = decltype(CI)::value * CH, n = NP - c0 < CH ? NP - c0 : CH;
      u32x4 pk[n];
      const u64* ps[n];
#pragma unroll
      for (int i = 0; i < n; ++i) ps[i] = src[c0 + i];
      WideLoads<n>::run(pk, ps);
#pragma unroll
      for (int i = 0; i < n; ++i)
        if ((pending & (1u << (c0 + i))) && pk[i].y == epoch && pk[i].w == epoch) {
          *reinterpret_cast<float2*>(dst + 2 * (t + (c0 + i) * NT)) = make_float2(__uint_as_float(pk[i].x), __uint_as_float(pk[i].z));
          pending &= ~(1u << (c0 + i));
        }
    });
    if (pending) {
      ++spins;
      if (spins > spin_limit || bail_flag() ||
          ((spins & 255u) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
        sh.bail = 1;
        atomicCAS(err, 0, (int)epoch);
        break;
      }
    }
  }
}

// The same for NQ words of three values (publish3). CPW = 0: word q carries values 3q .. 3q + 2 of dst. Otherwise
// every producer owns CPW consecutive values of dst and publishes them as ceil(CPW / 3) words, the last one padded.
template <int NQ, int CPW>
__device__ __forceinline__ void poll_triples(const u64* __restrict__ buf, unsigned epoch, float* dst, int* err, int delay,
                                             unsigned spin_limit) {
  constexpr int NP = (NQ + NT - 1) / NT;
  constexpr int CH = 7;
  constexpr int T = (CPW + 2) / 3;
  const int t = opaque(threadIdx.x);
  unsigned pending = 0;
  const u64* src[NP];
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const bool mine = i * NT + NT <= NQ || t + i * NT < NQ;
    if (mine) pending |= 1u << i;
    src[i] = buf + 2 * (mine ? t + i * NT : NQ - 1);
  }
  unsigned spins = 0;
  nap(delay);
  while (pending) {
    static_for<(NP + CH - 1) / CH>([&](auto CI) {
      constexpr int c0 = decltype(CI)::value * CH, n = NP - c0 < CH ? NP - c0 : CH;
      u32x4 pk[n];
      const u64* ps[n];
#pragma unroll
      for (int i = 0; i < n; ++i) ps[i] = src[c0 + i];
      WideLoads<n>::run(pk, ps);
#pragma unroll
      for (int i = 0; i < n; ++i)
        if ((pending & (1u << (c0 + i))) && pk[i].w == epoch) {
          const int q = t + (c0 + i) * NT;
          if constexpr (CPW % 3 == 0) {
            float* d = dst + 3 * q;
            d[0] = __uint_as_float(pk[i].x);
            d[1] = __uint_as_float(pk[i].y);
            d[2] = __uint_as_float(pk[i].z);
          } else {
            const int pw = q / T, r = q - pw * T;
            float* d = dst + pw * CPW + 3 * r;
            d[0] = __uint_as_float(pk[i].x);
            if (3 * r + 1 < CPW) d[1] = __uint_as_float(pk[i].y);
            if (3 * r + 2 < CPW) d[2] = __uint_as_float(pk[i].z);
          }
          pending &= ~(1u << (c0 + i));
        }
    });
    if (pending) {
      ++spins;
      if (spins > spin_limit || bail_flag() ||
          ((spins & 255u) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)) {
        sh.bail = 1;
        atomicCAS(err, 0, (int)epoch);
        break;
      }
    }
  }
}

// Registers of one linear phase: this wave's share of the weight slab (MAXI items per lane).
template <int MAXI, bool I8>
struct WSet {
  typename std::conditional<I8, int, float4>::type w[MAXI];  // an int8 item is one word per lane
};

// Per-layer column parameters of a workgroup in LDS: bias of local column c of phase ph at
// colp[ph * LPW + c], int8 column scale / 127 at colp[(4 + ph) * LPW + c]. They are requested
// into one register per thread a phase before the layer starts and deposited next to the
// layer's first input row; build_colparams lays them out per layer and workgroup. (Held in registers of the finishing lanes for the length of a
// phase they were the first values the compiler spilled, and a spill of a value just
// requested waits for every load in flight, the weights of the next phase included.)
constexpr int LPW = PD_COLP / 8;  // columns of a phase per workgroup, at most

constexpr bool LN_EPILOGUE = true;
// Linear phases of a layer, in execution order.
enum { PH_QKV = 0, PH_PROJ = 1, PH_FC = 2, PH_FC2 = 3 };

// Bias and int8 scale of local column c of phase ph, read ahead of the dot products (any lane may ask:
// c wraps inside the phase's LPW slots).
struct ColParams {
  float bias, scale;
};
template <bool SECOND>
__device__ __forceinline__ ColParams col_params(const float* colp, int ph, int c) {
  c &= LPW - 1;
  ColParams r;
  r.bias = colp[ph * LPW + c];
  r.scale = SECOND ? colp[(4 + ph) * LPW + c] : 1.f;
  return r;
}
// A column behind a folded LayerNorm (fp32 slabs hold diag(gamma) W, the bias holds bias + beta W, and the second
// slot the column sum S = sum_k gamma_k W_kc): with the row's mean and reciprocal standard deviation
// sum_k ((x_k - mean) rstd) gamma_k W_kc = rstd (dot - mean S), so the statistics are reduced side by side with the
// dot products instead of in two dependent reductions in front of them.
__device__ __forceinline__ float finish_ln(float dot, float mean, float rstd, const ColParams& cp) {
  return rstd * (dot - mean * cp.scale) + cp.bias;
}
// int8 items behind a LayerNorm (gemv_whole_ln8): gsum = sum_k gamma_k q_kn, scale the column scale / 127, and the
// bias holds bias_n + scale sum_k beta_k q_kn.
__device__ __forceinline__ float finish_ln8(float dot, float mean, float rstd, const ColParams& cp, float gsum) {
  return (rstd * (dot - mean * gsum)) * cp.scale + cp.bias;
}
// Finished value of a column from its dot product: the int8 column scale, the bias last.
template <bool I8>
__device__ __forceinline__ float finish(float dot, const ColParams& cp) {
  return (I8 ? dot * cp.scale : dot) + cp.bias;
}


// The four signed bytes of a word as floats (element e in bits 8e..8e+7,
// other/int8-gemm.js:36-43).
__device__ __forceinline__ float4 bytes_to_float4(int w) {
  return make_float4((float)((w << 24) >> 24), (float)((w << 16) >> 24), (float)((w << 8) >> 24), (float)(w >> 24));
}

// Calls f(std::integral_constant<int, wave>) so that everything derived from the
// wave index is a compile-time constant inside f (one copy of the code per wave).
template <class F>
__device__ __forceinline__ void for_wave(int wave, F f) {
  switch (wave) {
    case 0: f(std::integral_constant<int, 0>()); break;
    case 1: f(std::integral_constant<int, 1>()); break;
    case 2: f(std::integral_constant<int, 2>()); break;
    case 3: f(std::integral_constant<int, 3>()); break;
    case 4: f(std::integral_constant<int, 4>()); break;
    case 5: f(std::integral_constant<int, 5>()); break;
    case 6: f(std::integral_constant<int, 6>()); break;
    default: f(std::integral_constant<int, 7>()); break;
  }
}

__device__ __forceinline__ int ld_stream(const int* p) { return __builtin_nontemporal_load(p); }
template <bool RESIDENT>
__device__ __forceinline__ float4 ld_table(const float4* p) { return RESIDENT ? *p : ld_stream(p); }
__device__ __forceinline__ void zero_item(float4& v) { v = make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ void zero_item(int& v) { v = 0; }
__device__ __forceinline__ float4 to_float4(const float4& v) { return v; }
__device__ __forceinline__ float4 to_float4(int v) { return bytes_to_float4(v); }
// One item's contribution to a running sum. int8 items (whose phases are bound by their vector instructions: four
// conversions per word) take four chained multiply-adds, fp32 items two products, two multiply-adds and two additions.
template <bool CHAIN>
__device__ __forceinline__ float item_sum(float acc, const float4& w, const float4& x) {
  if constexpr (CHAIN) return __builtin_fmaf(w.w, x.w, __builtin_fmaf(w.z, x.z, __builtin_fmaf(w.y, x.y, __builtin_fmaf(w.x, x.x, acc))));
  else return acc + ((w.x * x.x + w.y * x.y) + (w.z * x.z + w.w * x.w));
}


template <class P>
struct KSplit {
  static constexpr int SW = (P::S + NW - 1) / NW;  // segments per wave
  static constexpr int IPW = SW * P::CPW;          // items per wave
};

// Layouts of a wave's share of a phase: whole columns, runs of consecutive items, segments of every column.
enum { LAY_WHOLE = 0, LAY_RUNS = 1, LAY_KSPLIT = 2 };

// Requests this wave's items of the workgroup's slab share into registers, one item per call; item
// j = c * S + seg of the workgroup is 64 consecutive lanes' worth (a float4, or one word of four int8,
// per lane) of segment seg of local column c. `ncols` is the number of columns this workgroup
// finishes (CPW except at the ragged end). A call costs the wave the time the memory pipeline takes
// to accept the request (several clocks per request and wave, the eight waves queueing for one
// pipeline), so the requests of the next phase are dealt out between the dot products of the current
// one instead of standing in front of them.
template <class P, int LAYOUT, class WS, class T>
struct ItemLoader {
  static constexpr int N = LAYOUT == LAY_KSPLIT ? KSplit<P>::IPW : P::IPW;
  WS& ws;
  const T* wgbase;  // this lane's word of the workgroup's first item
  int ncols, wave;
  // int8 columns whose length is no multiple of an item's 256 rows end in an item of zeros beyond row K: its lanes
  // beyond K request nothing (1600 rows stored as 7 items: an eighth of the bytes of such a matrix)
  static constexpr bool TAIL = std::is_same<T, int>::value && LAYOUT == LAY_WHOLE && P::K % SEG != 0;
  bool tail_live;   // this lane has rows of the last item
  __device__ __forceinline__ ItemLoader(WS& ws_, const T* slab, int ncols_, int wg, int wave_, int lane)
      : ws(ws_), wgbase(slab + (size_t)wg * P::ITEMS * 64 + opaque(lane)), ncols(ncols_), wave(wave_),
        tail_live(!TAIL || lane * 4 < P::K - (P::S - 1) * SEG) {}
  template <int I>
  __device__ __forceinline__ void item() const {
    if constexpr (LAYOUT == LAY_WHOLE) {
      constexpr int cc = I / P::S, seg = I % P::S;
      const int c = wave + cc * NW;
      if constexpr (!P::RAGGED && P::CPW % NW == 0) {
        ws.w[I] = ld_stream(wgbase + (c * P::S + seg) * 64);
      } else {
        zero_item(ws.w[I]);
        if (c < (P::RAGGED ? ncols : P::CPW) && (!TAIL || seg != P::S - 1 || tail_live)) ws.w[I] = ld_stream(wgbase + (c * P::S + seg) * 64);
      }
    } else if constexpr (LAYOUT == LAY_RUNS) {
      // unconditional: what lies beyond the share re-reads its last item and is never used
      int j = wave * P::IPW + I;
      j = j < P::ITEMS ? j : P::ITEMS - 1;
      ws.w[I] = ld_stream(wgbase + j * 64);
    } else {
      // unconditional: a wave beyond the last segment re-reads it (and multiplies it with zeros), the
      // slab holds zeros for the columns a workgroup at the ragged end does not have
      constexpr int si = I / P::CPW, c = I % P::CPW;
      int seg = wave + si * NW;
      seg = seg < P::S ? seg : P::S - 1;
      ws.w[I] = ld_stream(wgbase + (c * P::S + seg) * 64);
    }
  }
  // the items of slot J when the N requests are dealt out over NS slots
  template <int J, int NS>
  __device__ __forceinline__ void slot() const {
    constexpr int B = J * N / NS, E = (J + 1) * N / NS;
    static_for<E - B>([&](auto k) { this->template item<B + decltype(k)::value>(); });
  }
  // All of them at once (the code of a run of requests is shorter than that of the same requests one by one).
  __device__ __forceinline__ void all() const { part<0, 1>(); }
  // A compute unit's memory pipeline takes requests for about 32 KB without holding the waves (measured with
  // all 256 compute units requesting at once: 16 KB 33 clocks, 32 KB 190, 48 KB 540, 64 KB 1330, 96 KB 2500):
  // a phase whose share is larger is requested in two halves (whole columns, or runs of items), the second
  // when the phase has published.
  static constexpr bool HALVES = LAYOUT != LAY_KSPLIT && P::ITEMS * (int)sizeof(T) * 64 > 24 * 1024 &&
                                 (LAYOUT == LAY_WHOLE ? P::CW >= 2 : P::IPW >= 2);
  // Part H of NH: of the whole columns of this wave, or of its run of items.
  template <int H, int NH>
  __device__ __forceinline__ void part() const {
    if constexpr (LAYOUT == LAY_WHOLE) {
#pragma unroll
      for (int cc = P::CW * H / NH; cc < P::CW * (H + 1) / NH; ++cc) {
        const int c = wave + cc * NW;
#pragma unroll
        for (int seg = 0; seg < P::S; ++seg) zero_item(ws.w[cc * P::S + seg]);
        if (c < (P::RAGGED ? ncols : P::CPW)) {
#pragma unroll
          for (int seg = 0; seg < P::S; ++seg)
            if (!TAIL || seg != P::S - 1 || tail_live) ws.w[cc * P::S + seg] = ld_stream(wgbase + (c * P::S + seg) * 64);
        }
      }
    } else if constexpr (LAYOUT == LAY_RUNS) {
      const int nitems = ncols * P::S;
      for_wave(wave, [&](auto W) {
        constexpr int J0 = decltype(W)::value * P::IPW;
#pragma unroll
        for (int i = P::IPW * H / NH; i < P::IPW * (H + 1) / NH; ++i) {
          zero_item(ws.w[i]);
          if (J0 + i < P::ITEMS) {
            if (!P::RAGGED || J0 + i < nitems) ws.w[i] = ld_stream(wgbase + (J0 + i) * 64);
          }
        }
      });
    } else {
      static_assert(NH == 1, "the segment layout is requested whole or item by item");
      static_for<N>([&](auto k) { this->template item<decltype(k)::value>(); });
    }
  }
  // at the start of the phase before / after that phase has published
  __device__ __forceinline__ void early() const {
    if constexpr (HALVES) part<0, 2>();
    else all();
  }
  __device__ __forceinline__ void late() const {
    if constexpr (HALVES) part<1, 2>();
  }
};

// Of a share that is dealt out between dot products, only the first NUM/DEN (the rest is requested when the
// phase has published: `rest`).
template <class L, int NUM, int DEN>
struct Leading {
  static constexpr int NE = L::N * NUM / DEN;
  const L& l;
  template <int J, int NS>
  __device__ __forceinline__ void slot() const {
    constexpr int B = J * NE / NS, E = (J + 1) * NE / NS;
    static_for<E - B>([&](auto k) { l.template item<B + decltype(k)::value>(); });
  }
  __device__ __forceinline__ void rest() const {
    static_for<L::N - NE>([&](auto k) { l.template item<NE + decltype(k)::value>(); });
  }
};

// What a dot-product loop calls after item J of its NS when nothing is to be requested.
struct NoRequests {
  template <int J, int NS>
  __device__ __forceinline__ void slot() const {}
};
// Keeps the requests where they were written: the scheduler would otherwise move them all to the front.
template <class R>
__device__ __forceinline__ void pin_requests() {
  if constexpr (!std::is_same<R, NoRequests>::value) __builtin_amdgcn_sched_barrier(0);
}

// LayerNorm parameters travel global memory -> registers (requested with the weights
// of the phase) -> LDS (deposited next to the polled input row, before the barrier
// that follows the poll): gamma at lnp[0, D), beta at lnp[D, 2D).
// GAMMA_ONLY: a LayerNorm that is taken as an epilogue of int8 items needs no beta (it is in the folded bias).
template <int D, bool GAMMA_ONLY = false, int NLN>
__device__ __forceinline__ void request_ln(float4 (&r)[NLN], const float* __restrict__ gamma, const float* __restrict__ beta) {
  const int t = opaque(threadIdx.x);
#pragma unroll
  for (int i = 0; i < NLN; ++i) {
    const int idx = t + i * NT;
    if (GAMMA_ONLY && i * NT >= D / 4) continue;
    r[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (idx < D / 4) r[i] = reinterpret_cast<const float4*>(gamma)[idx];
    else if (!GAMMA_ONLY && idx < D / 2) r[i] = reinterpret_cast<const float4*>(beta)[idx - D / 4];
  }
}
template <int D, bool GAMMA_ONLY = false, int NLN>
__device__ __forceinline__ void deposit_ln(const float4 (&r)[NLN], float* lnp) {
  const int t = opaque(threadIdx.x);
#pragma unroll
  for (int i = 0; i < NLN; ++i)
    if (t + i * NT < (GAMMA_ONLY ? D / 4 : D / 2)) reinterpret_cast<float4*>(lnp)[t + i * NT] = r[i];
}

// The input row (LDS, zero padded up to S * SEG) as this lane's float4 of every
// segment; with LNORM normalised first (instructions.js:451-550: biased variance
// about the mean, eps inside the square root). Every wave derives the two
// statistics itself, so the LayerNorm needs no barrier. AFFINE applies gamma and
// beta from lnp; without it the caller's weights hold diag(gamma) W and its bias
// holds bias + beta W (eight waves re-reading 2*K parameters from LDS every phase
// cost about a microsecond per LayerNorm).
template <int K, bool LNORM, bool AFFINE>
__device__ __forceinline__ void input_row(float4 (&xr)[(K + SEG - 1) / SEG], const float* xs, const float* lnp, int lane) {
  constexpr int S = (K + SEG - 1) / SEG;
  const int l4 = opaque(lane) * 4;
#pragma unroll
  for (int s2 = 0; s2 < S; ++s2) xr[s2] = *reinterpret_cast<const float4*>(xs + s2 * SEG + l4);
  if (LNORM) {
    float sum = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < S; ++s2) sum += (xr[s2].x + xr[s2].y) + (xr[s2].z + xr[s2].w);
    const float mean = wave_sum(sum) * (1.0f / (float)K);
    float q = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < S; ++s2) {
      // lanes beyond K hold zeros that must not count as (0 - mean)^2
      const bool in = s2 * SEG + SEG <= K || s2 * SEG + lane * 4 < K;
      xr[s2].x -= mean; xr[s2].y -= mean; xr[s2].z -= mean; xr[s2].w -= mean;
      const float qq = (xr[s2].x * xr[s2].x + xr[s2].y * xr[s2].y) + (xr[s2].z * xr[s2].z + xr[s2].w * xr[s2].w);
      q += in ? qq : 0.f;
    }
    const float rstd = fast_rsqrt(wave_sum(q) * (1.0f / (float)K) + 1e-5f);
#pragma unroll
    for (int s2 = 0; s2 < S; ++s2) {
      const bool in = s2 * SEG + SEG <= K || s2 * SEG + lane * 4 < K;
      if (AFFINE) {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        const float4 g = in ? *reinterpret_cast<const float4*>(lnp + s2 * SEG + l4) : z;
        const float4 b = in ? *reinterpret_cast<const float4*>(lnp + K + s2 * SEG + l4) : z;
        xr[s2].x = g.x * (xr[s2].x * rstd) + b.x;
        xr[s2].y = g.y * (xr[s2].y * rstd) + b.y;
        xr[s2].z = g.z * (xr[s2].z * rstd) + b.z;
        xr[s2].w = g.w * (xr[s2].w * rstd) + b.w;
      } else {
        // gamma and beta live in the weights and the bias; padding lanes meet zero weights
        xr[s2].x *= rstd; xr[s2].y *= rstd; xr[s2].z *= rstd; xr[s2].w *= rstd;
      }
    }
  }
}

// The same row with gamma and beta applied (shapes that cannot fold them into their weights), as a joint
// effort of the workgroup: thread t owns float4 t of the row. Each wave sums its 256 elements and their
// squared distances from the wave's own mean; after a barrier every thread merges the NW pairs the same
// way (mean = sum of sums / K; sum of squares about it = sum_w q_w + n_w (m_w - mean)^2, the two-pass
// result without a second exchange), finishes its float4 and leaves it in xn (an LDS row nobody reads in
// this phase); after a second barrier every wave takes the finished row from there. `red` is 2 * NW
// floats of LDS scratch. (Every wave deriving the statistics of the whole row and re-reading 2*K
// parameters cost three microseconds per LayerNorm at K = 1600.)
template <int K>
__device__ __forceinline__ void input_row_shared(float4 (&xr)[(K + SEG - 1) / SEG], const float* xs, const float* lnp, float* xn,
                                                 float* red, int wave, int lane) {
  constexpr int S = (K + SEG - 1) / SEG;
  static_assert(K % 4 == 0 && S * 64 <= NT, "a thread owns one float4 of the row");
  const int t = opaque(threadIdx.x);
  const bool own = t < K / 4;
  const int tc = t < S * 64 ? t : S * 64 - 1;  // threads beyond the row read its zero padding
  const float4 x = reinterpret_cast<const float4*>(xs)[tc];
  int nw = K - wave * SEG;  // elements of the row in this wave
  nw = nw < 0 ? 0 : (nw > SEG ? SEG : nw);
  const float sw = wave_sum((x.x + x.y) + (x.z + x.w));
  const float mw = nw > 0 ? sw * (1.0f / (float)nw) : 0.f;
  const float dx = x.x - mw, dy = x.y - mw, dz = x.z - mw, dw = x.w - mw;
  const float qw = wave_sum(own ? (dx * dx + dy * dy) + (dz * dz + dw * dw) : 0.f);
  if (lane == 0) {
    red[wave] = sw;
    red[NW + wave] = qw;
  }
  __syncthreads();
  float sums[NW], qs[NW];
#pragma unroll
  for (int v = 0; v < NW; v += 4) {
    *reinterpret_cast<float4*>(sums + v) = *reinterpret_cast<const float4*>(red + v);
    *reinterpret_cast<float4*>(qs + v) = *reinterpret_cast<const float4*>(red + NW + v);
  }
  float total = 0.f;
#pragma unroll
  for (int v = 0; v < NW; ++v) total += sums[v];
  const float mean = total * (1.0f / (float)K);
  float m2 = 0.f;
#pragma unroll
  for (int v = 0; v < NW; ++v) {
    const int nv = K - v * SEG < 0 ? 0 : (K - v * SEG > SEG ? SEG : K - v * SEG);
    if (nv > 0) {
      const float d = sums[v] * (1.0f / (float)nv) - mean;
      m2 += qs[v] + (float)nv * (d * d);
    }
  }
  const float rstd = fast_rsqrt(m2 * (1.0f / (float)K) + 1e-5f);
  if (t < S * 64) {
    float4 y = make_float4(0.f, 0.f, 0.f, 0.f);
    if (own) {
      const float4 g = reinterpret_cast<const float4*>(lnp)[t];
      const float4 b = reinterpret_cast<const float4*>(lnp + K)[t];
      y = make_float4(g.x * ((x.x - mean) * rstd) + b.x, g.y * ((x.y - mean) * rstd) + b.y,
                      g.z * ((x.z - mean) * rstd) + b.z, g.w * ((x.w - mean) * rstd) + b.w);
    }
    reinterpret_cast<float4*>(xn)[t] = y;
  }
  __syncthreads();
  const int l4 = opaque(lane) * 4;
#pragma unroll
  for (int s2 = 0; s2 < S; ++s2) xr[s2] = *reinterpret_cast<const float4*>(xn + s2 * SEG + l4);
}

// WHOLE phases: the dot products of this wave's columns; lane cc returns the sum of
// the wave's cc-th column (local column wave + cc * NW), before scale and bias. `next` requests
// its items between the items of this phase.
template <class P, bool LNORM, bool AFFINE, class WS, class R = NoRequests>
__device__ __forceinline__ float gemv_whole(const WS& ws, const float* xs, const float* lnp, int ncols, int wave, int lane,
                                            float* xn = nullptr, float* red = nullptr, const R& next = R()) {
  static_assert(P::WHOLE, "phase is not laid out by whole columns");
  // a normalised row is held in registers; a plain one is read from LDS item by item
  float4 xr[LNORM ? P::S : 1];
  if constexpr (LNORM && AFFINE) input_row_shared<P::K>(reinterpret_cast<float4(&)[(P::K + SEG - 1) / SEG]>(xr), xs, lnp, xn, red, wave, lane);
  else if constexpr (LNORM) input_row<P::K, LNORM, AFFINE>(reinterpret_cast<float4(&)[(P::K + SEG - 1) / SEG]>(xr), xs, lnp, lane);
  const float* xl = xs + opaque(lane) * 4;
  float val = 0.f;
  static_for<P::CW>([&](auto CC) {
    constexpr int cc = decltype(CC)::value;
    const bool valid = wave + cc * NW < (P::RAGGED ? ncols : P::CPW);
    float acc = 0.f;
    auto item = [&](auto SG) {
      constexpr int seg = decltype(SG)::value;
      const float4 x = LNORM ? xr[LNORM ? seg : 0] : *reinterpret_cast<const float4*>(xl + seg * SEG);
      const float4 w = to_float4(ws.w[cc * P::S + seg]);
      acc = item_sum<std::is_same<decltype(ws.w[0] + 0), int>::value>(acc, w, x);
    };
    if constexpr (std::is_same<R, NoRequests>::value) {
      if (valid) static_for<P::S>(item);
    } else {
      static_for<P::S>([&](auto SG) {
        if (valid) item(SG);
        next.template slot<cc * P::S + decltype(SG)::value, P::CW * P::S>();
        pin_requests<R>();
      });
    }
    if (valid) {
      const float r = wave_sum(acc);
      val = lane == cc ? r : val;
    }
  });
  return val;
}

// WHOLE phases behind a folded LayerNorm: the raw row against the wave's columns, and the row's sum and sum of
// squares in the same reduction; lane cc returns the dot product of the wave's cc-th column, every lane the mean
// and the reciprocal standard deviation (instructions.js:451-550: biased variance, eps inside the square root).
template <class P, class WS>
__device__ __forceinline__ float gemv_whole_ln(const WS& ws, const float* xs, int ncols, int wave, int lane, float& mean, float& rstd) {
  static_assert(P::WHOLE, "phase is not laid out by whole columns");
  const int l4 = opaque(lane) * 4;
  float4 xr[P::S];
#pragma unroll
  for (int s2 = 0; s2 < P::S; ++s2) xr[s2] = *reinterpret_cast<const float4*>(xs + s2 * SEG + l4);  // (zero beyond K)
  float red[2 + P::CW];
  red[0] = 0.f;
  red[1] = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < P::S; ++s2) {
    red[0] += (xr[s2].x + xr[s2].y) + (xr[s2].z + xr[s2].w);
    red[1] += (xr[s2].x * xr[s2].x + xr[s2].y * xr[s2].y) + (xr[s2].z * xr[s2].z + xr[s2].w * xr[s2].w);
  }
  static_for<P::CW>([&](auto CC) {
    constexpr int cc = decltype(CC)::value;
    const bool valid = wave + cc * NW < (P::RAGGED ? ncols : P::CPW);
    float acc = 0.f;
    if (valid) static_for<P::S>([&](auto SG) {
      constexpr int seg = decltype(SG)::value;
      acc = item_sum<false>(acc, to_float4(ws.w[cc * P::S + seg]), xr[seg]);
    });
    red[2 + cc] = acc;
  });
  wave_sum_n(red);
  mean = red[0] * (1.0f / (float)P::K);
  const float var = fmaxf(__builtin_fmaf(-mean, mean, red[1] * (1.0f / (float)P::K)), 0.f);
  rstd = fast_rsqrt(var + 1e-5f);
  float val = 0.f;
#pragma unroll
  for (int cc = 0; cc < P::CW; ++cc) val = lane == cc ? red[2 + cc] : val;
  return val;
}

// The same behind a LayerNorm whose gamma is not in the weights (int8 items): the raw row times gamma (gam: LDS,
// gamma followed by beta, so that a read beyond K meets finite values; the row is zero there) against the wave's
// columns, the statistics of the raw row in the same reduction. sum_k ((x_k - mean) rstd gamma_k + beta_k) q_kn =
// rstd (dot - mean G_n) + sum_k beta_k q_kn with dot = sum_k x_k gamma_k q_kn and G_n = sum_k gamma_k q_kn: the
// caller finishes with G_n and a bias that holds the beta term (fold_ln_i8_kernel). `next` requests its items
// between the items of this phase.
template <class P, class WS, class R>
__device__ __forceinline__ float gemv_whole_ln8(const WS& ws, const float* xs, const float* gam, int ncols, int wave, int lane,
                                                float& mean, float& rstd, const R& next) {
  static_assert(P::WHOLE, "phase is not laid out by whole columns");
  const int l4 = opaque(lane) * 4;
  float4 xr[P::S];
  float red[2 + P::CW];
  red[0] = 0.f;
  red[1] = 0.f;
#pragma unroll
  for (int s2 = 0; s2 < P::S; ++s2) {
    const float4 x = *reinterpret_cast<const float4*>(xs + s2 * SEG + l4);  // (zero beyond K)
    const float4 g = *reinterpret_cast<const float4*>(gam + s2 * SEG + l4);
    red[0] += (x.x + x.y) + (x.z + x.w);
    red[1] += (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
    xr[s2] = make_float4(x.x * g.x, x.y * g.y, x.z * g.z, x.w * g.w);
  }
  static_for<P::CW>([&](auto CC) {
    constexpr int cc = decltype(CC)::value;
    const bool valid = wave + cc * NW < (P::RAGGED ? ncols : P::CPW);
    float acc = 0.f;
    static_for<P::S>([&](auto SG) {
      constexpr int seg = decltype(SG)::value;
      if (valid) acc = item_sum<true>(acc, to_float4(ws.w[cc * P::S + seg]), xr[seg]);
      next.template slot<cc * P::S + seg, P::CW * P::S>();
      pin_requests<R>();
    });
    red[2 + cc] = acc;
  });
  wave_sum_n(red);
  mean = red[0] * (1.0f / (float)P::K);
  const float var = fmaxf(__builtin_fmaf(-mean, mean, red[1] * (1.0f / (float)P::K)), 0.f);
  rstd = fast_rsqrt(var + 1e-5f);
  float val = 0.f;
#pragma unroll
  for (int cc = 0; cc < P::CW; ++cc) val = lane == cc ? red[2 + cc] : val;
  return val;
}

// Other phases: per (column, wave) partial sums go to part[col * NW + wave]. The item
// code exists once per wave with every index a constant: a phase is short, and what
// it costs is instruction count (a runtime-indexed single copy measured 5-15 %
// slower at d = 1280 and 1600).
template <class P, class WS, class R = NoRequests>
__device__ __forceinline__ void gemv_split(const WS& ws, const float* xs, float* part, int ncols, int wave, int lane,
                                           const R& next = R()) {
  static_assert(!P::WHOLE, "phase is laid out by whole columns");
  constexpr int S = P::S;
  const float* xl = xs + opaque(lane) * 4;
  const int nitems = ncols * S;
  for_wave(wave, [&](auto W) {
    constexpr int WV = decltype(W)::value;
    constexpr int J0 = WV * P::IPW;
    float acc = 0.f;
    static_for<P::IPW>([&](auto II) {
      constexpr int i = decltype(II)::value;
      if constexpr (J0 + i < P::ITEMS) {
        if (!P::RAGGED || J0 + i < nitems) {
          constexpr int seg = (J0 + i) % S, col = (J0 + i) / S;
          const float4 x = *reinterpret_cast<const float4*>(xl + seg * SEG);
          const float4 w = to_float4(ws.w[i]);
          acc += (w.x * x.x + w.y * x.y) + (w.z * x.z + w.w * x.w);
          if (seg == S - 1 || i == P::IPW - 1 || J0 + i == P::ITEMS - 1) {
            const float r = wave_sum(acc);
            if (lane == 0) part[col * NW + WV] = r;
            acc = 0.f;
          }
        }
      }
      next.template slot<i, P::IPW>();
      pin_requests<R>();
    });
  });
}

// The long contraction split along K instead (shapes whose whole kernel sits at the register limit, where
// the compiler fetches a row segment from LDS per item and waits for each): wave w takes segments
// w, w + NW, ... of every column of the workgroup, so a segment is fetched once for CPW items; the
// per-wave partial of column c goes to part[c * NW + w] and thread c adds the NW of them in wave order.
template <class P, class WS, class R = NoRequests>
__device__ __forceinline__ void gemv_ksplit(const WS& ws, const float* xs, float* part, int wave, int lane, const R& next = R()) {
  const float* xl = xs + opaque(lane) * 4;
  float acc[P::CPW];
#pragma unroll
  for (int c = 0; c < P::CPW; ++c) acc[c] = 0.f;
  static_for<KSplit<P>::SW>([&](auto SI) {
    constexpr int si = decltype(SI)::value;
    const int seg = wave + si * NW;
    const int segc = seg < P::S ? seg : P::S - 1;
    float4 x = *reinterpret_cast<const float4*>(xl + segc * SEG);
    if (seg >= P::S) x = make_float4(0.f, 0.f, 0.f, 0.f);
    static_for<P::CPW>([&](auto CI) {
      constexpr int c = decltype(CI)::value;
      const float4 w = to_float4(ws.w[si * P::CPW + c]);
      acc[c] = item_sum<std::is_same<decltype(ws.w[0] + 0), int>::value>(acc[c], w, x);
      next.template slot<si * P::CPW + c, KSplit<P>::IPW>();
      pin_requests<R>();
    });
  });
  wave_sum_n(acc);
#pragma unroll
  for (int c = 0; c < P::CPW; ++c)
    if (lane == 0) part[c * NW + wave] = acc[c];
}
template <class P>
__device__ __forceinline__ float column_sum_ksplit(const float* part, int c) {
  float s = 0.f;
#pragma unroll
  for (int v = 0; v < NW; ++v) s += part[c * NW + v];
  return s;
}

// Sum of the per-wave partials of local column c, in ascending wave order.
template <class P>
__device__ __forceinline__ float column_sum(const float* part, int c) {
  const int v0 = (c * P::S) / P::IPW;
  int v1 = ((c + 1) * P::S - 1) / P::IPW;
  v1 = v1 > NW - 1 ? NW - 1 : v1;
  float s = 0.f;
  for (int v = v0; v <= v1; ++v) s += part[c * NW + v];
  return s;
}


#ifdef WGPT_TRACE
#define TRACE(slot)                                                                              \
  do {                                                                                           \
    if (a.trace && tid == 0 && step == a.nsteps - 1) a.trace[(size_t)wg * 512 + (slot)] = wall_clock64(); \
  } while (0)
#define TRACE5(k)                                                                                 \
  do {                                                                                            \
    if (a.trace && tid == 0 && step == a.nsteps - 1 && li == 5) a.trace[(size_t)wg * 512 + 400 + PH * 16 + (k)] = wall_clock64(); \
  } while (0)
#else
#define TRACE(slot) do {} while (0)
#define TRACE5(k) do {} while (0)
#endif

// Order of selectTopK (globals.js:66-74): larger logit first, lower index first among equals;
// index INT_MAX marks an empty candidate.
constexpr int NOCAND = 0x7fffffff;
__device__ __forceinline__ bool cand_before(float ov, int oi, float cv, int ci) {
  return oi != NOCAND && (ci == NOCAND || ov > cv || (ov == cv && oi < ci));
}
// The first candidate of the wave in that order, as wave-uniform values.
__device__ __forceinline__ void wave_first(float& v, int& i) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(v, off);
    const int oi = __shfl_xor(i, off);
    if (cand_before(ov, oi, v, i)) {
      v = ov;
      i = oi;
    }
  }
}


constexpr int cmax(int a, int b) { return a > b ? a : b; }

template <class C>
struct Phases {
  typedef Phase<3 * C::D, C::D, true> A;    // c_attn
  typedef Phase<C::D, C::D, true> Cc;       // attention c_proj
  typedef Phase<C::HID, C::D, true> Dd;     // c_fc
  typedef Phase<C::D, C::HID, false> E;     // mlp c_proj
  static constexpr bool EKS = C::I8;        // ... split along the contraction (see KSplit)
  static constexpr int MAXI = cmax(cmax(A::IPW, Dd::IPW), cmax(Cc::IPW, EKS ? KSplit<E>::IPW : E::IPW));
  // Two register sets (c_attn and c_fc in one, the two projections in the other) let a
  // phase's weights be requested a whole phase ahead, right after the poll of the
  // phase before it; affordable while a set is at most 32 registers.
  static constexpr bool DUAL = MAXI * (C::I8 ? 1 : 4) <= 32;
  // With two sets the next phase's requests stand either in front of the current phase's work (its
  // LayerNorm and dot products then wait until the memory pipeline has accepted them) or between
  // its dot products (they then reach memory later, and the next poll, whose answer returns in
  // order behind them, may see its words late). Short phases want the first, long ones the second.
  static constexpr bool SPREAD = DUAL && C::I8;
};

// SAMPLE: top-k selection and sampling in the kernel (top_k in 2..PD_TOPK); the arg-max kernel
// stays free of its registers.
// Floats of dynamic LDS the phases use (rows, staged exchange words, partial sums, parameter blocks), rounded to
// a multiple of four so that what follows is 16-byte aligned.
template <class C>
constexpr int lds_floats() {
  typedef Phases<C> PS;
  constexpr int XS = (C::SD + C::SH) * SEG;
  constexpr int ATTP = C::ATTW > 2 * PD_TOPK * C::G ? C::ATTW : 2 * PD_TOPK * C::G;
  constexpr int PART = 32 * (C::HS + 4) > PS::E::CPW * NW ? 32 * (C::HS + 4) : PS::E::CPW * NW;
  return (XS + 2 * C::D + ATTP + PART + 3 * C::HS + PS::A::CPW + 2 * PS::Cc::CPW + PS::Dd::CPW + PD_COLP + 16 + 3) / 4 * 4;
}
// Rows of the vocabulary table a workgroup keeps in the LDS its phases leave free, for the whole launch: the
// first rows of its run, a multiple of the wave count, at most one batch of the vocabulary loop. A compute unit
// has 160 KB; 2 KB stay aside for the static part.
constexpr int PD_VOCAB_BATCH = 4;  // rows of wte in flight per wave
template <class C>
constexpr int table_rows_in_lds() {
  constexpr int spare = (160 * 1024 - 2048) / 4 - lds_floats<C>();
  // the wider shapes sit at the register limit, lose more to the extra code than the few rows that fit would give
  // them (d = 1280: 0.784 against 0.779 ms/token, int8 d = 1600: 1.00 against 0.80), and keep none
  constexpr int rows = (spare > 0 && C::D <= PD_NARROW_D && !C::I8) ? spare / C::D / NW * NW : 0;
  return rows > NW * PD_VOCAB_BATCH ? NW * PD_VOCAB_BATCH : rows;
}

// Rows per wave that stay in registers next to them (12 registers a row at d = 768; with the candidate lists of
// top-k sampling a fourth row would spill).
template <class C, bool SAMPLE>
constexpr int table_rows_in_registers() {
  return (table_rows_in_lds<C>() > 0 && C::D <= 768) ? (SAMPLE ? 3 : 4) : 0;
}

template <class C, int MAXKV, bool SAMPLE>
__global__ __launch_bounds__(NT) void decode_persistent_kernel(PersistentArgs a) {
  typedef Phases<C> PS;
  typedef typename PS::A PA;
  typedef typename PS::Cc PC;
  typedef typename PS::Dd PD;
  typedef typename PS::E PE;
  constexpr int D = C::D, HS = C::HS, H = C::H, HID = C::HID, SPLIT = C::SPLIT, MAXI = PS::MAXI;
  constexpr bool DUAL = PS::DUAL, I8 = C::I8, EKS = PS::EKS, SPREAD = PS::SPREAD;
  constexpr int SPN = 2, SPD = 3;  // share of a dealt-out request run that goes between the dot products
  constexpr bool FOLD = !I8;  // fp32 slabs carry the LayerNorm gamma, their biases the beta (see build_slab, fold_ln_bias)
  // hidden row and attention slices exchanged as words of three values (the fp32 d = 1600 shape, which lives on spilled
  // registers, spills five times as much with them and keeps {value, epoch} pairs)
  constexpr bool TRIPLE_H = I8 || D < 1600, TRIPLE_ATT = TRIPLE_H;
  // ... and the LayerNorm in front of c_attn and c_fc is an epilogue of the dot products (finish_ln; the fp32 d = 1600
  // shape spills six times as much with it)
  constexpr bool LNEPI = FOLD && LN_EPILOGUE && D <= 1280;
  // int8 items: the same with gamma multiplied into the row instead of into the weights (gemv_whole_ln8). The column
  // sums ride in the free slots of the projections' bias rows of colp (build_colparams_kernel).
  constexpr bool LNEPI8 = I8 && LN_EPILOGUE;
  static_assert(!LNEPI8 || (PC::CPW + PD::CPW <= LPW && PE::CPW + PA::CPW <= LPW), "no room for the column sums in colp");
  constexpr int XS0 = C::SD * SEG;                                  // floats of a D-long input row
  constexpr int XS1 = C::SH * SEG;                                  // floats of a HID-long input row
  constexpr int ATTP = C::ATTW > 2 * PD_TOPK * C::G ? C::ATTW : 2 * PD_TOPK * C::G;  // floats of the staged exchange words
  constexpr int PART = 32 * (HS + 4) > PE::CPW * NW ? 32 * (HS + 4) : PE::CPW * NW;
  constexpr int NLN = (D / 2 + NT - 1) / NT;                        // float4 of LayerNorm parameters per thread

  // Input rows alternate between two buffers (xs0: residual stream rows; xs1: merged
  // attention output, MLP hidden row), so that a poll never writes the buffer the
  // dot products of the phase before it may still be reading.
  // 16-byte aligned behind the static part (676 bytes): a 128-bit LDS access at an address that is not a
  // multiple of 16 is split by the hardware and takes several times as long
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* xs0 = lds;            // [XS0]
  float* xs1 = xs0 + XS0;      // [XS1]
  float* lnp = xs1 + XS1;      // [2*D] LayerNorm gamma, beta of the next normalising phase
  float* attp = lnp + 2 * D;   // [ATTP]
  float* part = attp + ATTP;   // [PART]
  float* qkv_s = part + PART;  // [3*HS]
  static_assert(FOLD || (XS0 + XS1 + 2 * D + ATTP) % 4 == 0, "part is read as float4 by the cooperative LayerNorm");
  float* pubA = qkv_s + 3 * HS;   // [PA::CPW] finished c_attn columns
  float* pubC = pubA + PA::CPW;   // [PC::CPW] residual stream after the attention projection
  float* pubD = pubC + PC::CPW;   // [PD::CPW] finished c_fc columns
  float* colp = pubD + PD::CPW + PE::CPW;   // [8 * LPW] biases and int8 column scales of this workgroup's columns of the layer
  static_assert(PA::CPW <= LPW && PC::CPW <= LPW && PD::CPW <= LPW && PE::CPW <= LPW, "a phase has more columns per workgroup than colp holds");
  // Launches of several steps keep the first LROWS rows of the workgroup's run of the vocabulary table here
  // from start to end: that share of the table is read from memory once per launch instead of once per token.
  constexpr int LROWS = table_rows_in_lds<C>(), LR = LROWS / NW;
  // the host takes the last step's logits from its pinned buffer for exactly these shapes (persistent_writes_host_logits),
  // and the kernel writes them there only where it keeps table rows: the two must not drift apart
  static_assert((LROWS > 0) == (!I8 && D <= PD_NARROW_D), "host-side and kernel-side conditions for host logits differ");
  static_assert(LROWS == 0 || (PD_GRID * 4 * D >= 50257 && XS1 >= 4 * D), "a workgroup's run of logits is staged in the hidden row's buffer");
  float* vres = lds + lds_floats<C>();  // [LROWS * D]

  const int wg = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: same for the whole wave
  if (tid == 0) {
    sh.bail = 0;
    // a misaligned row buffer would only be slow, not wrong: report it instead of running at a third of the speed
    if ((reinterpret_cast<size_t>(lds) & 15u) != 0) atomicCAS(a.err, 0, -16);
  }
  for (int e = tid; e < XS0 + XS1; e += NT) lds[e] = 0.f;  // the padding of xs0 beyond D stays zero for good

  // columns this workgroup finishes per phase (fewer than CPW only at the ragged end)
  auto cols_of = [&](int N, int CPW) {
    const int n = N - wg * CPW;
    return n > CPW ? CPW : (n < 0 ? 0 : n);
  };
  const int ncA = cols_of(PA::N, PA::CPW), ncC = cols_of(PC::N, PC::CPW);
  const int ncD = cols_of(PD::N, PD::CPW), ncE = cols_of(PE::N, PE::CPW);
  // local column this lane finishes (lane cc of wave v: column v + cc * NW)
  const int fc = wave + lane * NW;
  const bool finA = lane < PA::CW && fc < ncA, finC = lane < PC::CW && fc < ncC, finD = lane < PD::CW && fc < ncD;

  // attention role: head and slice of the positions; threads form 32 key groups
  // (tid >> 4) of 16 lanes (tid & 15)
  const bool att_role = wg < H * SPLIT;
  const int ah = wg / SPLIT, as = wg - ah * SPLIT;

  const LayerParamOffsets po = layer_param_offsets(D);
  typedef WSet<MAXI, I8> WS;
  WS ws0, ws1;
  WS& wX = ws0;                // c_attn, c_fc
  WS& wY = DUAL ? ws1 : ws0;   // attention c_proj, mlp c_proj
  float4 lnreg[NLN];
  typedef typename std::conditional<I8, int, float4>::type Item;
  const Item* slabs = reinterpret_cast<const Item*>(a.slabs);
  typedef ItemLoader<PA, LAY_WHOLE, WS, Item> LoadA;
  typedef ItemLoader<PC, LAY_WHOLE, WS, Item> LoadC;
  typedef ItemLoader<PD, LAY_WHOLE, WS, Item> LoadD;
  typedef ItemLoader<PE, EKS ? LAY_KSPLIT : LAY_RUNS, WS, Item> LoadE;
  float4 kreg[MAXKV], vreg[MAXKV];
  unsigned ep = a.ebase;
  int tok = a.tok ? a.tok[0] : a.tok_value;

  // the layer's block for this workgroup is already in the layout of colp (build_colparams): one load per thread
  float preg = 0.f;
  auto request_params = [&](int layer) {
    // unconditional (the upper half of the workgroup re-reads the lower half's words): after a load
    // under a branch the compiler waits for every load in flight where the paths join
    preg = a.colparams[((size_t)layer * PD_GRID + wg) * PD_COLP + (opaque(tid) & (PD_COLP - 1))];
  };
  auto deposit_params = [&]() {
    const int t = opaque(tid);
    if (t < PD_COLP) colp[t] = preg;
  };
  // (not for a table so small that these rows would be most of the run: loading them then costs more than it saves)
  const int lrows = (LROWS > 0 && a.nsteps >= PD_TABLE_LDS_STEPS && a.rows_per_wg >= 4 * LROWS) ? LROWS : 0;
  if (lrows) {
    const int v0 = wg * a.rows_per_wg;
    for (int e = tid; e < LROWS * (D / 4); e += NT) {
      const int r = e / (D / 4), c = e - r * (D / 4);
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (r < a.rows_per_wg && v0 + r < a.V) v = reinterpret_cast<const float4*>(a.wte + (size_t)(v0 + r) * D)[c];
      reinterpret_cast<float4*>(vres)[e] = v;
    }
  }
  // ... and the RROWS rows behind them in registers the narrow shapes leave free, RR per wave
  constexpr int RR = table_rows_in_registers<C, SAMPLE>(), RROWS = RR * NW;
  [[maybe_unused]] float4 wres[RR > 0 ? RR : 1][C::SD];
  if constexpr (RR > 0) {
    if (lrows) {
      const int ln = opaque(tid & 63);
      const int vb = wg * a.rows_per_wg + LROWS + wave * RR;
#pragma unroll
      for (int r = 0; r < RR; ++r)
#pragma unroll
        for (int s2 = 0; s2 < C::SD; ++s2) {
          wres[r][s2] = make_float4(0.f, 0.f, 0.f, 0.f);
          if (LROWS + wave * RR + r < a.rows_per_wg && vb + r < a.V && (s2 * SEG + SEG <= D || s2 * SEG + ln * 4 < D))
            wres[r][s2] = *reinterpret_cast<const float4*>(a.wte + (size_t)(vb + r) * D + s2 * SEG + ln * 4);
        }
    }
  }
  const int rrows = (RR > 0 && lrows) ? RROWS : 0;
  request_params(0);
  LoadA(wX, slabs, ncA, wg, wave, lane).all();
  deposit_params();
  // FOLD: only the final LayerNorm has parameters, and they stay in lnp for good
  if (FOLD) request_ln<D>(lnreg, a.lnf_g, a.lnf_b);
  else request_ln<D>(lnreg, a.lparams + po.ln1g, a.lparams + po.ln1b);
  deposit_ln<D>(lnreg, lnp);
  __syncthreads();

  for (int step = 0; step < a.nsteps; ++step) {
    const int pos = a.pos0 + step;
    TRACE(0);
#ifdef WGPT_TRACE
    if (a.trace && tid == 0 && step == a.nsteps - 1) a.trace[(size_t)wg * 512 + 500] = __builtin_readcyclecounter();
#endif
    // ---- embedding: every workgroup builds the row itself (instructions.js:795-821) ----
    for (int e = tid; e < D; e += NT) xs0[e] = a.wte[(size_t)tok * D + e] + a.wpe[(size_t)pos * D + e];
    if (step > 0) deposit_params();  // the first layer's, requested during the last layer of the token before
    __syncthreads();

    // slice of positions 0..pos for the attention role
    const int nkeys = pos + 1;
    const int chunk = (nkeys + SPLIT - 1) / SPLIT;
    const int c0 = as * chunk;
    int c1 = c0 + chunk;
    c1 = c1 > nkeys ? nkeys : c1;
    const bool has_new = pos >= c0 && pos < c1;  // this slice holds the new position
    const int nkv = c1 > c0 ? (c1 - c0 + 31) / 32 : 0;  // key batches of this slice

    float own_r = 0.f;  // residual stream value of the column this lane finishes in the attention projection

    for (int li = 0; li < a.L; ++li) {
      const Item* slab = slabs + (size_t)li * a.slab_stride;
      const float* lp = a.lparams + (size_t)li * po.stride;
      float* Kc = a.kv + ((size_t)(li * 2 + 0) * H + ah) * a.ctx * HS;
      float* Vc = a.kv + ((size_t)(li * 2 + 1) * H + ah) * a.ctx * HS;

      // ======================= c_attn: LN1 + QKV =======================
      {
        [[maybe_unused]] constexpr int PH = PH_QKV;
        if (li > 0) {
          poll_words<D>(a.bufR2, ep, xs0, a.err, a.delay[0], a.spin_limit);
          if (!FOLD) deposit_ln<D, LNEPI8>(lnreg, lnp);
          deposit_params();
          __syncthreads();
          if (sh.bail) return;
        }
        wait_loads();
        TRACE(1 + li * 8 + PH);
        const LoadC nextC(wY, slab + a.slab_offC, ncC, wg, wave, lane);
        if (DUAL && !SPREAD) nextC.early();
        own_r = finC ? xs0[wg * PC::CPW + fc] : 0.f;
        const ColParams cp = col_params<true>(colp, PH, fc);  // second slot: int8 scale, or the column sum of a folded LayerNorm
        float dot, mean = 0.f, rstd = 1.f;
        if constexpr (SPREAD && LNEPI8) dot = gemv_whole_ln8<PA>(wX, xs0, lnp, ncA, wave, lane, mean, rstd, nextC);
        else if constexpr (SPREAD) dot = gemv_whole<PA, true, !FOLD>(wX, xs0, lnp, ncA, wave, lane, xs1, part, nextC);
        else if constexpr (LNEPI) dot = gemv_whole_ln<PA>(wX, xs0, ncA, wave, lane, mean, rstd);
        else dot = gemv_whole<PA, true, !FOLD>(wX, xs0, lnp, ncA, wave, lane, xs1, part);
        TRACE5(2);
        if (finA) {
          if constexpr (SPREAD && LNEPI8) pubA[fc] = finish_ln8(dot, mean, rstd, cp, colp[PH_FC2 * LPW + ((PE::CPW + fc) & (LPW - 1))]);
          else pubA[fc] = LNEPI ? finish_ln(dot, mean, rstd, cp) : finish<I8>(dot, cp);
        }
        __syncthreads();
        ++ep;
        if (tid < ncA) publish(a.bufQKV + wg * PA::CPW + tid, pubA[tid], ep);
        TRACE5(4);
        if (!DUAL) nextC.all();
        else if (!SPREAD) nextC.late();
        TRACE5(5);
        if (att_role) {
          // this layer's cached keys and values of the slice
          const int g16 = opaque(tid >> 4), sub = opaque(tid & 15);
#pragma unroll
          for (int i = 0; i < MAXKV; ++i) {
            const int j = c0 + g16 + 32 * i;
            float4 kk = make_float4(0.f, 0.f, 0.f, 0.f), vv = kk;
            if (i < nkv && j < c1 && j < pos) {
              // Ordinary 128-bit loads (half the instructions of 64-bit agent-scope ones). A row is complete at
              // agent scope before any workgroup can reach a token that reads it (see the wait before the
              // end-of-token publish), it never changes afterwards, and no line of it is read before it is written
              // (j < pos; a 128-byte line holds part of one row only): no cache can hold a stale copy of it.
              // (The fp32 d = 1600 shape, which lives on spilled registers, keeps the 64-bit form: 1.556 against
              // 1.877 ms/token with these.)
              if constexpr (I8 || D < 1600) {
                kk = *reinterpret_cast<const float4*>(Kc + (size_t)j * HS + sub * 4);
                vv = *reinterpret_cast<const float4*>(Vc + (size_t)j * HS + sub * 4);
              } else {
                const u64* kp = reinterpret_cast<const u64*>(Kc + (size_t)j * HS + sub * 4);
                const u64* vp = reinterpret_cast<const u64*>(Vc + (size_t)j * HS + sub * 4);
                const u64 k0 = ld_word(kp), k1 = ld_word(kp + 1), v0 = ld_word(vp), v1 = ld_word(vp + 1);
                kk = make_float4(__uint_as_float((unsigned)k0), __uint_as_float((unsigned)(k0 >> 32)),
                                 __uint_as_float((unsigned)k1), __uint_as_float((unsigned)(k1 >> 32)));
                vv = make_float4(__uint_as_float((unsigned)v0), __uint_as_float((unsigned)(v0 >> 32)),
                                 __uint_as_float((unsigned)v1), __uint_as_float((unsigned)(v1 >> 32)));
              }
            }
            kreg[i] = kk;
            vreg[i] = vv;
          }
        }
        TRACE5(6);
      }

      // ======================= attention slice (role workgroups) =======================
      ++ep;  // epoch of the attention outputs
      if (att_role) {
        {
          unsigned pending = tid < 3 * HS ? 1u : 0u;
          unsigned spins = 0;
          nap(a.delay[1]);
          const int which = tid / HS, e = tid - which * HS;
          const u64* src = a.bufQKV + which * D + ah * HS + e;
          while (pending) {
            const u64 pk = ld_word(src);
            if ((unsigned)(pk >> 32) == ep - 1) {
              qkv_s[tid] = __uint_as_float((unsigned)pk);
              pending = 0;
            } else if (++spins > a.spin_limit || bail_flag()) {
              sh.bail = 1;
              atomicCAS(a.err, 0, (int)ep);
              break;
            }
          }
        }
        __syncthreads();
        wait_loads();
        TRACE(1 + li * 8 + 5);
        // the slice that holds the new position appends it to the cache and uses it from LDS
        if (has_new && tid < 32) {
          const float* src = qkv_s + (tid < 16 ? HS : 2 * HS) + (tid & 15) * 4;
          float* dstp = (tid < 16 ? Kc : Vc) + (size_t)pos * HS + (tid & 15) * 4;
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
          sc[i] = -INFINITY;
          if (i < nkv) {
            const int j = c0 + g16 + 32 * i;
            if (j == pos && has_new) {
              kreg[i] = *reinterpret_cast<const float4*>(qkv_s + HS + sub * 4);
              vreg[i] = *reinterpret_cast<const float4*>(qkv_s + 2 * HS + sub * 4);
            }
            const float p = row16_sum((qv.x * kreg[i].x + qv.y * kreg[i].y) + (qv.z * kreg[i].z + qv.w * kreg[i].w));
            sc[i] = j < c1 ? p * a.scale : -INFINITY;
            m = fmaxf(m, sc[i]);
          }
        }
        // softmax numerators against the maximum of this group of 16 lanes (its keys only)
        float l = 0.f;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int i = 0; i < MAXKV; ++i) {
          if (i < nkv) {
            const float p = sc[i] > -INFINITY ? fast_exp(sc[i] - m) : 0.f;
            l += p;
            o.x += p * vreg[i].x; o.y += p * vreg[i].y; o.z += p * vreg[i].z; o.w += p * vreg[i].w;
          }
        }
        // the four groups of a wave combine in registers (rescaled to the wave's maximum) ...
        float mw = xor16_max(m);
        mw = xor32_max(mw);
        const float f = m > -INFINITY ? fast_exp(m - mw) : 0.f;
        l *= f;
        o.x *= f; o.y *= f; o.z *= f; o.w *= f;
        l = xor16_sum(l); o.x = xor16_sum(o.x); o.y = xor16_sum(o.y); o.z = xor16_sum(o.z); o.w = xor16_sum(o.w);
        l = xor32_sum(l); o.x = xor32_sum(o.x); o.y = xor32_sum(o.y); o.z = xor32_sum(o.z); o.w = xor32_sum(o.w);
        // ... and the eight waves through LDS: (o[HS], m, l) per wave
        if (lane < 16) {
          *reinterpret_cast<float4*>(part + wave * (HS + 4) + sub * 4) = o;
          if (sub == 0) {
            part[wave * (HS + 4) + HS] = mw;
            part[wave * (HS + 4) + HS + 1] = l;
          }
        }
        __syncthreads();
        if constexpr (!TRIPLE_ATT) {
          if (tid < HS + 2) {
            float M = -INFINITY;
#pragma unroll
            for (int w2 = 0; w2 < NW; ++w2) M = fmaxf(M, part[w2 * (HS + 4) + HS]);
            float v = M;
            if (tid != HS) {
              const int c = tid < HS ? tid : HS + 1;
              v = 0.f;
#pragma unroll
              for (int w2 = 0; w2 < NW; ++w2) {
                const float mv = part[w2 * (HS + 4) + HS];
                v += part[w2 * (HS + 4) + c] * (mv > -INFINITY ? fast_exp(mv - M) : 0.f);
              }
            }
            publish(a.bufATT + (size_t)wg * (HS + 2) + tid, v, ep);
          }
        } else if (wave == 0) {
          // Wave 0 combines the eight: lane l takes element l of the output, lanes of equal l & 7 the factor
          // exp(m_w - M) of wave w = l & 7 (one exponential per lane instead of eight in a row per element).
          static_assert(HS == 64 && NW == 8, "one lane per element, eight waves");
          const int lw = lane & (NW - 1);
          const float mv = part[lw * (HS + 4) + HS];
          const float M = group8_max(mv);
          const float f = mv > -INFINITY ? fast_exp(mv - M) : 0.f;
          const float lsum = group8_sum(part[lw * (HS + 4) + HS + 1] * f);
          float o = 0.f;
#pragma unroll
          for (int w2 = 0; w2 < NW; ++w2)
            o += part[w2 * (HS + 4) + lane] * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), w2));
          // (o[0..63], M, l) as 22 words of three values: word r = values 3r .. 3r + 2
          const float a0 = __shfl(o, 3 * lane), a1 = __shfl(o, 3 * lane + 1), a2 = __shfl(o, 3 * lane + 2);
          const bool lastw = lane == (HS + 2) / 3 - 1;
          if (lane < (HS + 2) / 3)
            publish3(a.bufATT + 2 * ((size_t)wg * ((HS + 2) / 3) + lane), a0, lastw ? M : a1, lastw ? lsum : a2, ep);
        }
      }

      // ======================= attention c_proj: merge slices, project, residual =======================
      {
        [[maybe_unused]] constexpr int PH = PH_PROJ;
        const int att_delay = att_role ? a.delay[2] + ((pos * a.att_slope[0]) >> 10) : a.delay[3] + ((pos * a.att_slope[1]) >> 10);
        if constexpr (TRIPLE_ATT) poll_triples<C::ATTW / 3, 0>(a.bufATT, ep, attp, a.err, att_delay, a.spin_limit);
        else poll_words<C::ATTW>(a.bufATT, ep, attp, a.err, att_delay, a.spin_limit);
        __syncthreads();
        wait_loads();
        TRACE(1 + li * 8 + PH);
        const LoadD nextD(wX, slab + a.slab_offD, ncD, wg, wave, lane);
        if (DUAL && !SPREAD) nextD.early();
        if (DUAL && !FOLD) request_ln<D, LNEPI8>(lnreg, lp + po.ln2g, lp + po.ln2b);
        // merge of the slices of each head (flash-decoding): element e of head h is
        // sum_s o_s[e] exp(m_s - M) / sum_s l_s exp(m_s - M), M = max_s m_s. The H * SPLIT normalised weights
        // exp(m_s - M) / sum are made once (thread h * SPLIT + s; `part` is idle between the attention and the
        // next LayerNorm) and read back as broadcasts: every element deriving them itself cost SPLIT exponentials
        // per element, 1.45 us of the phase at d = 1600.
        // (The fp32 d = 1600 shape, which lives on spilled registers, keeps the per-element form: with the extra
        // barrier and the shared weights it ran 8 % slower, 1.585 -> 1.713 ms/token.)
        constexpr int MERGE_ROUNDS = (D + NT - 1) / NT;
        constexpr bool MERGE_ONCE = I8 || D < 1600;
        static_assert(H * SPLIT <= NT && H * SPLIT <= PART, "one thread and one float of `part` per (head, slice)");
        if (MERGE_ONCE && tid < H * SPLIT) {
          const int h = tid / SPLIT;
          const float* phd = attp + h * SPLIT * (HS + 2);
          float ms[SPLIT];
          float M = -INFINITY;
#pragma unroll
          for (int s2 = 0; s2 < SPLIT; ++s2) {
            ms[s2] = phd[s2 * (HS + 2) + HS];
            M = fmaxf(M, ms[s2]);
          }
          float Lsum = 0.f, mine = 0.f;
#pragma unroll
          for (int s2 = 0; s2 < SPLIT; ++s2) {
            const float wv = ms[s2] > -INFINITY ? fast_exp(ms[s2] - M) : 0.f;
            Lsum += phd[s2 * (HS + 2) + HS + 1] * wv;
            mine = s2 == tid - h * SPLIT ? wv : mine;
          }
          part[tid] = mine * fast_rcp(Lsum);
        }
        if (MERGE_ONCE) __syncthreads();
        const Leading<LoadD, SPN, SPD> leadD{nextD};
        static_for<MERGE_ROUNDS>([&](auto KK) {
          constexpr int k = decltype(KK)::value;
          const int e = tid + k * NT;
          if (k * NT + NT <= D || e < D) {
            const int h = e / HS, c = e - h * HS;
            const float* phd = attp + h * SPLIT * (HS + 2);
            if constexpr (MERGE_ONCE) {
              const float* wn = part + h * SPLIT;
              float val = 0.f;
#pragma unroll
              for (int s2 = 0; s2 < SPLIT; ++s2) val += phd[s2 * (HS + 2) + c] * wn[s2];
              xs1[e] = val;
            } else {
              float ms[SPLIT];
              float M = -INFINITY;
#pragma unroll
              for (int s2 = 0; s2 < SPLIT; ++s2) {
                ms[s2] = phd[s2 * (HS + 2) + HS];
                M = fmaxf(M, ms[s2]);
              }
              float Lsum = 0.f, val = 0.f;
#pragma unroll
              for (int s2 = 0; s2 < SPLIT; ++s2) {
                const float wv = ms[s2] > -INFINITY ? fast_exp(ms[s2] - M) : 0.f;
                Lsum += phd[s2 * (HS + 2) + HS + 1] * wv;
                val += phd[s2 * (HS + 2) + c] * wv;
              }
              xs1[e] = val * fast_rcp(Lsum);
            }
          }
          // (the few dot products of this phase cannot take c_fc's requests between them: the rounds of the merge do)
          if constexpr (SPREAD) {
            leadD.template slot<k, MERGE_ROUNDS>();
            __builtin_amdgcn_sched_barrier(0);
          }
        });
        if (XS0 > D) {  // the hidden row of the layer before reached into the padding
          for (int e = D + tid; e < XS0; e += NT) xs1[e] = 0.f;
        }
        __syncthreads();
        TRACE5(1);
        const ColParams cp = col_params<I8>(colp, PH, fc);
        float dot;
        dot = gemv_whole<PC, false, false>(wY, xs1, lnp, ncC, wave, lane);
        TRACE5(2);
        if (finC) pubC[fc] = own_r + finish<I8>(dot, cp);  // model.js:159
        __syncthreads();
        ++ep;
        if (tid < ncC) publish(a.bufR1 + wg * PC::CPW + tid, pubC[tid], ep);
        TRACE5(4);
        if (!DUAL) {
          nextD.all();
          if (!FOLD) request_ln<D, LNEPI8>(lnreg, lp + po.ln2g, lp + po.ln2b);
        } else if (!SPREAD) nextD.late();
        else leadD.rest();
        TRACE5(5);
      }

      // ======================= c_fc: LN2 + fc + GELU =======================
      {
        [[maybe_unused]] constexpr int PH = PH_FC;
        poll_words<D>(a.bufR1, ep, xs0, a.err, a.delay[4], a.spin_limit);
        if (!FOLD) deposit_ln<D, LNEPI8>(lnreg, lnp);
        __syncthreads();
        wait_loads();
        TRACE(1 + li * 8 + PH);
        const LoadE nextE(wY, slab + a.slab_offE, ncE, wg, wave, lane);
        if (DUAL && !SPREAD) nextE.early();
        const ColParams cp = col_params<true>(colp, PH, fc);
        float dot, mean = 0.f, rstd = 1.f;
        const Leading<LoadE, SPN, SPD> leadE{nextE};
        if constexpr (SPREAD && LNEPI8) dot = gemv_whole_ln8<PD>(wX, xs0, lnp, ncD, wave, lane, mean, rstd, leadE);
        else if constexpr (SPREAD) dot = gemv_whole<PD, true, !FOLD>(wX, xs0, lnp, ncD, wave, lane, xs1, part, leadE);
        else if constexpr (LNEPI) dot = gemv_whole_ln<PD>(wX, xs0, ncD, wave, lane, mean, rstd);
        else dot = gemv_whole<PD, true, !FOLD>(wX, xs0, lnp, ncD, wave, lane, xs1, part);
        TRACE5(2);
        if (finD) {  // model.js:188
          if constexpr (SPREAD && LNEPI8) pubD[fc] = gelu_ref(finish_ln8(dot, mean, rstd, cp, colp[PH_PROJ * LPW + ((PC::CPW + fc) & (LPW - 1))]));
          else pubD[fc] = gelu_ref(LNEPI ? finish_ln(dot, mean, rstd, cp) : finish<I8>(dot, cp));
        }
        __syncthreads();
        ++ep;
        if constexpr (!TRIPLE_H) {
          if (tid < ncD) publish(a.bufH + wg * PD::CPW + tid, pubD[tid], ep);
        } else {
          constexpr int T = (PD::CPW + 2) / 3;  // words of three values per workgroup, the last one padded
          static_assert(!PD::RAGGED, "every workgroup finishes CPW hidden units");
          if (tid < T) {
            const int c = 3 * opaque(tid);
            publish3(a.bufH + 2 * (wg * T + tid), pubD[c], c + 1 < PD::CPW ? pubD[c + 1] : 0.f, c + 2 < PD::CPW ? pubD[c + 2] : 0.f, ep);
          }
        }
        TRACE5(4);
        if (!DUAL) nextE.all();
        else if (!SPREAD) nextE.late();
        else leadE.rest();
        TRACE5(5);
      }

      // ======================= mlp c_proj: fc2 + residual =======================
      {
        [[maybe_unused]] constexpr int PH = PH_FC2;
        // weights of the phase after this one: the next layer's c_attn share with its
        // LayerNorm; after the last layer the final LayerNorm (and, with two register
        // sets, already the first layer's share for the next token)
        auto request_small = [&]() {
          if (li + 1 < a.L) {
            request_params(li + 1);
            if (!FOLD) request_ln<D, LNEPI8>(lnreg, lp + po.stride + po.ln1g, lp + po.stride + po.ln1b);
          } else {
            if (!FOLD) request_ln<D>(lnreg, a.lnf_g, a.lnf_b);
            if (step + 1 < a.nsteps) request_params(0);
          }
        };
        // (the last layer of the last step requests the first layer's share too and leaves it unused)
        const LoadA nextA(wX, li + 1 < a.L ? slab + a.slab_stride : slabs, ncA, wg, wave, lane);
        if constexpr (TRIPLE_H) poll_triples<PD_GRID * ((PD::CPW + 2) / 3), PD::CPW>(a.bufH, ep, xs1, a.err, a.delay[5], a.spin_limit);
        else poll_words<HID>(a.bufH, ep, xs1, a.err, a.delay[5], a.spin_limit);
        __syncthreads();
        wait_loads();
        TRACE(1 + li * 8 + PH);
        if (DUAL && !SPREAD && (li + 1 < a.L || step + 1 < a.nsteps)) nextA.early();
        if (DUAL) request_small();
        const ColParams cpe = col_params<I8>(colp, PH, tid);  // thread c finishes local column c
        if constexpr (EKS && SPREAD) gemv_ksplit<PE>(wY, xs1, part, wave, lane, nextA);
        else if constexpr (EKS) gemv_ksplit<PE>(wY, xs1, part, wave, lane);
        else if constexpr (SPREAD) gemv_split<PE>(wY, xs1, part, ncE, wave, lane, nextA);
        else gemv_split<PE>(wY, xs1, part, ncE, wave, lane);
        TRACE5(2);
        __syncthreads();
        ++ep;
        if (tid < ncE) {  // model.js:205
          const float dot = EKS ? column_sum_ksplit<PE>(part, tid) : column_sum<PE>(part, tid);
          const float r2 = pubC[tid] + finish<I8>(dot, cpe);
          publish(a.bufR2 + wg * PE::CPW + tid, r2, ep);
        }
        TRACE5(4);
        if (!DUAL) {
          request_small();
          if (li + 1 < a.L) nextA.all();
        } else if (!SPREAD && (li + 1 < a.L || step + 1 < a.nsteps)) nextA.late();
        TRACE5(5);
      }
    }

    // ======================= final LayerNorm + vocabulary projection =======================
    poll_words<D>(a.bufR2, ep, xs0, a.err, a.delay[0], a.spin_limit);
    if (!FOLD) deposit_ln<D>(lnreg, lnp);
    __syncthreads();
    if (sh.bail) return;
    wait_loads();
    TRACE(1 + a.L * 8);
    {
      constexpr int S = C::SD, R = PD_VOCAB_BATCH;  // rows of wte in flight per wave
      // A table of up to 160 MB is read with ordinary loads, so that it may stay in the 256 MB memory-side cache
      // from one token to the next while the layers' weights stream past it with non-temporal loads (117M, 154 MB:
      // 0.1574 -> 0.1545 ms/token); a larger one would only push itself out (345M, 206 MB: 0.400 -> 0.425 with
      // ordinary loads) and is streamed like the weights.
      constexpr bool WTE_RESIDENT = D <= 768;
      const int lane = opaque(tid & 63);
      const int v0 = wg * a.rows_per_wg;
      int v1 = v0 + a.rows_per_wg;
      v1 = v1 > a.V ? a.V : v1;
      // final LayerNorm of the row, in registers (each wave for itself)
      float4 xv[S];
      input_row<D, true, true>(xv, xs0, lnp, lane);
      float best = -INFINITY;
      int besti = 0x7fffffff;
      // top_k > 1: this wave's K best rows so far, in order; (lastv, lasti) is the K-th
      const int K = SAMPLE ? a.top_k : 1;
      constexpr int KL = SAMPLE ? PD_TOPK : 1;
      float tv[KL], lastv = -INFINITY;
      int ti[KL], lasti = NOCAND;
#pragma unroll
      for (int j = 0; j < KL; ++j) {
        tv[j] = -INFINITY;
        ti[j] = NOCAND;
      }
      // the last step's logits also go to the caller's pinned memory, through LDS (narrow shapes only)
      [[maybe_unused]] const bool to_host = LROWS > 0 && a.host_logits != nullptr && step == a.nsteps - 1;
      if constexpr (LROWS == 0) {
        // the shapes at the register limit keep this loop exactly as it was tuned: sharing the per-row code below
        // with them moved d = 1280 from 0.779 to 0.785 ms/token
        for (int vb = v0 + wave * R; vb < v1; vb += NW * R) {
          float4 w[R][S];
#pragma unroll
          for (int r = 0; r < R; ++r)
#pragma unroll
            for (int s2 = 0; s2 < S; ++s2) {
              w[r][s2] = make_float4(0.f, 0.f, 0.f, 0.f);
              if (vb + r < v1 && (s2 * SEG + SEG <= D || s2 * SEG + lane * 4 < D))
                w[r][s2] = ld_table<WTE_RESIDENT>(reinterpret_cast<const float4*>(a.wte + (size_t)(vb + r) * D + s2 * SEG + lane * 4));
            }
#pragma unroll
          for (int r = 0; r < R; ++r) {
            float acc = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < S; ++s2)
              acc += (w[r][s2].x * xv[s2].x + w[r][s2].y * xv[s2].y) + (w[r][s2].z * xv[s2].z + w[r][s2].w * xv[s2].w);
            const float s = wave_sum(acc);
            if (vb + r < v1) {
              if (lane == 0) a.logits[vb + r] = s;
              if (s > best || besti == 0x7fffffff) {
                best = s;
                besti = vb + r;
              }
              if (SAMPLE && cand_before(s, vb + r, lastv, lasti)) {
                // insert: carry the displaced candidate down the list
                float cv = s;
                int ci = vb + r;
#pragma unroll
                for (int j = 0; j < KL; ++j) {
                  if (j < K && cand_before(cv, ci, tv[j], ti[j])) {
                    const float sv = tv[j];
                    const int si = ti[j];
                    tv[j] = cv;
                    ti[j] = ci;
                    cv = sv;
                    ci = si;
                  }
                  if (j == K - 1) {
                    lastv = tv[j];
                    lasti = ti[j];
                  }
                }
              }
            }
          }
        }
      } else {
        // one finished row: logit, running arg-max (rows come in ascending order per wave: the first index wins a
        // tie), top-k candidates
        auto tally = [&](float s, int row) {
          if (lane == 0) {
            a.logits[row] = s;
            if (to_host) xs1[row - v0] = s;  // (free since the last layer's second MLP product)
          }
          if (s > best || besti == 0x7fffffff) {
            best = s;
            besti = row;
          }
          if (SAMPLE && cand_before(s, row, lastv, lasti)) {
            // insert: carry the displaced candidate down the list
            float cv = s;
            int ci = row;
#pragma unroll
            for (int j = 0; j < KL; ++j) {
              if (j < K && cand_before(cv, ci, tv[j], ti[j])) {
                const float sv = tv[j];
                const int si = ti[j];
                tv[j] = cv;
                ti[j] = ci;
                cv = sv;
                ci = si;
              }
              if (j == K - 1) {
                lastv = tv[j];
                lasti = ti[j];
              }
            }
          }
        };
        if constexpr (LROWS > 0) {
          if (lrows) {  // the lowest rows of the run, from LDS
#pragma unroll
            for (int r = 0; r < LR; ++r) {
              float acc = 0.f;
#pragma unroll
              for (int s2 = 0; s2 < S; ++s2)
                if (s2 * SEG + SEG <= D || s2 * SEG + lane * 4 < D) {
                  const float4 wl = *reinterpret_cast<const float4*>(vres + (wave * LR + r) * D + s2 * SEG + lane * 4);
                  acc += (wl.x * xv[s2].x + wl.y * xv[s2].y) + (wl.z * xv[s2].z + wl.w * xv[s2].w);
                }
              const float s = wave_sum(acc);
              if (v0 + wave * LR + r < v1) tally(s, v0 + wave * LR + r);
            }
          }
        }
        if constexpr (RR > 0) {
          if (rrows) {  // the next rows, from registers
#pragma unroll
            for (int r = 0; r < RR; ++r) {
              float acc = 0.f;
#pragma unroll
              for (int s2 = 0; s2 < S; ++s2)
                acc += (wres[r][s2].x * xv[s2].x + wres[r][s2].y * xv[s2].y) + (wres[r][s2].z * xv[s2].z + wres[r][s2].w * xv[s2].w);
              const float s = wave_sum(acc);
              if (v0 + LROWS + wave * RR + r < v1) tally(s, v0 + LROWS + wave * RR + r);
            }
          }
        }
        for (int vb = v0 + lrows + rrows + wave * R; vb < v1; vb += NW * R) {
          float4 w[R][S];
#pragma unroll
          for (int r = 0; r < R; ++r)
#pragma unroll
            for (int s2 = 0; s2 < S; ++s2) {
              w[r][s2] = make_float4(0.f, 0.f, 0.f, 0.f);
              if (vb + r < v1 && (s2 * SEG + SEG <= D || s2 * SEG + lane * 4 < D))
                w[r][s2] = ld_table<WTE_RESIDENT>(reinterpret_cast<const float4*>(a.wte + (size_t)(vb + r) * D + s2 * SEG + lane * 4));
            }
#pragma unroll
          for (int r = 0; r < R; ++r) {
            float acc = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < S; ++s2)
              acc += (w[r][s2].x * xv[s2].x + w[r][s2].y * xv[s2].y) + (w[r][s2].z * xv[s2].z + w[r][s2].w * xv[s2].w);
            const float s = wave_sum(acc);
            if (vb + r < v1) tally(s, vb + r);
          }
        }
      }
      if (lane == 0) {
        sh.red[wave] = best;
        sh.red_idx[wave] = __int_as_float(besti);
      }
      if (SAMPLE && lane < PD_TOPK) {
        float cvv = -INFINITY;
        int cii = NOCAND;
#pragma unroll
        for (int j = 0; j < KL; ++j)
          if (lane == j) {
            cvv = tv[j];
            cii = ti[j];
          }
        sh.cand_v[wave * PD_TOPK + lane] = cvv;
        sh.cand_i[wave * PD_TOPK + lane] = cii;
      }
      __syncthreads();
      ++ep;
      if constexpr (LROWS > 0) {
        // contiguous 256-byte stores per wave instead of 50257 single words crossing the bus; wave 0 stays out of it:
        // it waits for its memory operations below, in front of the publish
        if (to_host && wave > 0)
          for (int r = tid - 64; r < v1 - v0; r += NT - 64) a.host_logits[v0 + r] = xs1[r];
      }
      // Visibility of this token's cache rows to the next token. The slice that owned the new position appended k and v
      // of every layer with write-through device-scope stores issued by wave 0; wave 0 also publishes this workgroup's
      // word of the arg-max exchange below. Waiting here until every memory operation of the wave has completed
      // (vmcnt = 0; the stores are tens of microseconds old, so the wait is free) orders them before that publish, and
      // every workgroup polls every word of this exchange before it starts the next token: whoever reads these rows in a
      // later step (slice boundaries move with the position, so it may be another workgroup) does so after they reached
      // the level at which all compute units agree. Within the token the new row is read only by its writer, from LDS.
      if (wave == 0) wait_loads();
      if (SAMPLE) {
        // the workgroup's K best of its waves' candidates (one per lane of wave 0), published in order
        if (wave == 0) {
          float cv = sh.cand_v[lane];
          int ci = sh.cand_i[lane];
          float wv = -INFINITY;
          int wi = NOCAND;
          for (int r = 0; r < K; ++r) {
            float fv = cv;
            int fi = ci;
            wave_first(fv, fi);
            if (lane == r) {
              wv = fv;
              wi = fi;
            }
            if (ci == fi) {  // indices are unique: the owner retires its candidate
              cv = -INFINITY;
              ci = NOCAND;
            }
          }
          if (lane < PD_TOPK) {
            publish(a.bufAM + 2 * (wg * PD_TOPK + lane), wv, ep);
            publish(a.bufAM + 2 * (wg * PD_TOPK + lane) + 1, __int_as_float(wi), ep);
          }
        }
      } else if (tid == 0) {
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
    TRACE(2 + a.L * 8);
#ifdef WGPT_TRACE
    if (a.trace && tid == 0 && step == a.nsteps - 1) a.trace[(size_t)wg * 512 + 501] = __builtin_readcyclecounter();
#endif
    if (step + 1 < a.nsteps) {
      if (!DUAL) LoadA(wX, slabs, ncA, wg, wave, lane).all();
      if (!FOLD) request_ln<D>(lnreg, a.lparams + po.ln1g, a.lparams + po.ln1b);
    }
    // ======================= arg-max over the workgroups, finished by everyone =======================
    double ustep = 0.0;
    if (SAMPLE) {
      ustep = a.u[step];
      poll_words<2 * PD_TOPK * C::G>(a.bufAM, ep, attp, a.err, a.delay[6], a.spin_limit);
    } else {
      poll_words<2 * C::G>(a.bufAM, ep, attp, a.err, a.delay[6], a.spin_limit);
    }
    if (!FOLD && step + 1 < a.nsteps) deposit_ln<D>(lnreg, lnp);  // every wave is past the final LayerNorm: the arg-max words need all of them
    __syncthreads();
    if (sh.bail) return;
    TRACE(3 + a.L * 8);
    if (SAMPLE) {
      // Every wave of every workgroup selects the same K candidates in order (selectTopK), applies
      // cpuSoftmax in float64 and sampleFromDistribution with the step's draw (globals.js:47-74).
      // A workgroup's list arrives in order, so a lane only ever looks at the heads of its G/64 lists.
      const int K = a.top_k;
      constexpr int LPL = C::G / 64;  // workgroup lists per lane
      static_assert(C::G % 64 == 0, "workgroup lists are dealt to lanes evenly");
      float hv[LPL];
      int hi[LPL], hp[LPL];
#pragma unroll
      for (int jj = 0; jj < LPL; ++jj) {
        const int c = (lane + 64 * jj) * PD_TOPK;
        hp[jj] = 0;
        hv[jj] = attp[2 * c];
        hi[jj] = __float_as_int(attp[2 * c + 1]);
      }
      float myv = -INFINITY;  // lane r keeps the r-th selection
      int myi = NOCAND;
      for (int r = 0; r < K; ++r) {
        float fv = -INFINITY;
        int fi = NOCAND;
#pragma unroll
        for (int jj = 0; jj < LPL; ++jj)
          if (cand_before(hv[jj], hi[jj], fv, fi)) {
            fv = hv[jj];
            fi = hi[jj];
          }
        wave_first(fv, fi);
        if (lane == r) {
          myv = fv;
          myi = fi;
        }
        // the owner moves on to the next entry of that list
#pragma unroll
        for (int jj = 0; jj < LPL; ++jj)
          if (hi[jj] == fi && fi != NOCAND) {
            ++hp[jj];
            const int c = (lane + 64 * jj) * PD_TOPK + hp[jj];
            hv[jj] = hp[jj] < K ? attp[2 * c] : -INFINITY;
            hi[jj] = hp[jj] < K ? __float_as_int(attp[2 * c + 1]) : NOCAND;
          }
      }
      // lane r: exp((x_r - max) / temperature); then the sums in the reference's order on every lane
      const float first = __shfl(myv, 0);
      const double mye = myi != NOCAND ? exp(((double)myv - (double)first) / a.temperature) : 0.0;
      double sum = 0.0;
      for (int r = 0; r < K; ++r) sum = sum + __shfl(mye, r);
      double cum = 0.0;
      int pick = NOCAND, lastsel = 0;
      for (int r = 0; r < K; ++r) {
        const int si = __shfl(myi, r);
        if (si != NOCAND) {
          cum += __shfl(mye, r) / sum;
          lastsel = si;
          if (pick == NOCAND && ustep < cum) pick = si;
        }
      }
      tok = pick != NOCAND ? pick : lastsel;
      if (wg == 0 && tid == 0) a.out_tok[step] = tok;
    } else {
      float b = -INFINITY;
      int bi = 0x7fffffff;
      for (int w2 = lane; w2 < C::G; w2 += 64) {
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
  // Workgroup 0 is past the last exchange, so every workgroup has published its last word: the launch is complete
  // unless a wait has expired somewhere meanwhile, which the error word says.
  if (a.host_done && wg == 0 && tid == 0) *a.host_done = __hip_atomic_load(a.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// rowscale (may be null): the gamma of the LayerNorm in front of the matrix, folded in as
// diag(gamma) W.
__global__ void build_slab_kernel(const float* __restrict__ W, int ldw, int K, int N, int cpw, int S, size_t total,
                                  const float* __restrict__ rowscale, float4* __restrict__ slab) {
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
      if (k + e < K) v[e] = W[(size_t)(k + e) * ldw + col] * (rowscale ? rowscale[k + e] : 1.0f);
  slab[idx] = make_float4(v[0], v[1], v[2], v[3]);
}

// out[n] = bias[n] + sum_k beta[k] W[k][n]: the beta of the LayerNorm in front of the
// matrix, folded into the bias (accumulated in double, rounded once).
// colsum[n] = sum_k fl(gamma[k] W[k][n]): the sum of the column as the slab holds it (build_slab_kernel rounds the
// same products), for the LayerNorm taken as an epilogue (finish_ln).
__global__ void fold_ln_bias_kernel(const float* __restrict__ W, int ldw, int K, int N, const float* __restrict__ gamma,
                                    const float* __restrict__ beta, const float* __restrict__ bias, float* __restrict__ out,
                                    float* __restrict__ colsum) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  double acc = 0.0, sum = 0.0;
  for (int k = 0; k < K; ++k) {
    const float w = W[(size_t)k * ldw + n];
    acc += (double)beta[k] * (double)w;
    sum += (double)(w * gamma[k]);
  }
  out[n] = (float)((double)bias[n] + acc);
  colsum[n] = (float)sum;
}

__global__ void fold_ln_i8_kernel(const int32_t* __restrict__ Wq, int ldwq, int K, int N, const float* __restrict__ scale,
                                  const float* __restrict__ gamma, const float* __restrict__ beta, const float* __restrict__ bias,
                                  float* __restrict__ out_bias, float* __restrict__ gsum) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= N) return;
  double bq = 0.0, gq = 0.0;
  const int sh = 8 * (n & 3);
  for (int k = 0; k < K; ++k) {
    const int q = (int)(int8_t)(((unsigned)Wq[(size_t)k * ldwq + (n >> 2)] >> sh) & 0xffu);
    bq += (double)beta[k] * (double)q;
    gq += (double)gamma[k] * (double)q;
  }
  out_bias[n] = (float)((double)bias[n] + (double)(scale[n] / 127.0f) * bq);
  gsum[n] = (float)gq;
}

// int8: item (w, j = c*S + seg, lane) is one word holding rows k..k+3 (k = seg*256 + lane*4)
// of column w*cpw + c, gathered from the reference packing [K, N/4] (4 consecutive
// columns per word, other/int8-gemm.js:36-43).
__global__ void build_slab_i8_kernel(const int32_t* __restrict__ Wq, int ldwq, int K, int N, int cpw, int S, size_t total,
                                     int32_t* __restrict__ slab) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  const size_t it = idx >> 6;
  const int per_wg = cpw * S;
  const int w = (int)(it / per_wg), j = (int)(it - (size_t)w * per_wg);
  const int c = j / S, seg = j - c * S;
  const int col = w * cpw + c, k = seg * SEG + lane * 4;
  unsigned out = 0;
  if (col < N)
    for (int e = 0; e < 4; ++e)
      if (k + e < K) {
        const unsigned word = (unsigned)Wq[(size_t)(k + e) * ldwq + (col >> 2)];
        out |= ((word >> (8 * (col & 3))) & 0xffu) << (8 * e);
      }
  slab[idx] = (int32_t)out;
}

// One thread per float of the per-workgroup parameter blocks: out[(layer * G + wg) * PD_COLP + t].
__global__ void build_colparams_kernel(const float* __restrict__ lparams, int L, int d, int i8, PhaseGeom gA, PhaseGeom gC,
                                       PhaseGeom gD, PhaseGeom gE, float* __restrict__ out) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)L * PD_GRID * PD_COLP) return;
  const int t = (int)(idx % PD_COLP), wg = (int)((idx / PD_COLP) % PD_GRID), layer = (int)(idx / ((size_t)PD_COLP * PD_GRID));
  const int kind = t / (4 * LPW), ph = (t / LPW) & 3, c = t % LPW;
  const LayerParamOffsets po = layer_param_offsets(d);
  const PhaseGeom g = ph == PH_QKV ? gA : ph == PH_PROJ ? gC : ph == PH_FC ? gD : gE;
  // (int8: the two matrices behind a LayerNorm take their biases with beta folded in)
  const int off = ph == PH_QKV ? (kind ? po.sA : i8 ? po.fA : po.bA) : ph == PH_PROJ ? (kind ? po.sC : po.bC)
                : ph == PH_FC ? (kind ? po.sD : i8 ? po.fD : po.bD) : (kind ? po.sE : po.bE);
  const int col = wg * g.cpw + c;
  float v = 0.f;
  // second slot: int8 column scales, or for fp32 the column sums of the two matrices behind a LayerNorm
  if (c < g.cpw && col < g.N && (kind == 0 || i8 || ph == PH_QKV || ph == PH_FC)) {
    v = lparams[(size_t)layer * po.stride + off + col];
    if (kind && i8) v = v / 127.0f;  // other/int8-gemm.js:126-132 divides by 127 before the column scale is applied
  }
  // int8: the column sums sum_k gamma_k q_kn of those two matrices ride in the bias rows of the two projections, behind
  // their (few) columns: c_fc's in attn c_proj's row, c_attn's in mlp c_proj's (col_gsum)
  if (i8 && kind == 0 && (ph == PH_PROJ || ph == PH_FC2) && c >= g.cpw) {
    const PhaseGeom gg = ph == PH_PROJ ? gD : gA;
    const int c2 = c - g.cpw, col2 = wg * gg.cpw + c2;
    if (c2 < gg.cpw && col2 < gg.N) v = lparams[(size_t)layer * po.stride + (ph == PH_PROJ ? po.gD : po.gA) + col2];
  }
  out[idx] = v;
}

template <class C>
size_t lds_bytes_of() {
  const size_t need = sizeof(float) * (size_t)(lds_floats<C>() + table_rows_in_lds<C>() * C::D);
  // more than half of a compute unit's 160 KB, so that exactly one workgroup lives on each
  const size_t one_per_cu = 84 * 1024;
  return need > one_per_cu ? need : one_per_cu;
}

template <class C, int MAXKV>
hipError_t launch_kv(const PersistentArgs& a, hipStream_t s) {
  const size_t lds_bytes = lds_bytes_of<C>();
  static bool enabled = false;  // dynamic LDS size already raised for the two instantiations
  if (!enabled) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_persistent_kernel<C, MAXKV, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e == hipSuccess)
      e = hipFuncSetAttribute(reinterpret_cast<const void*>(decode_persistent_kernel<C, MAXKV, true>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
    if (e != hipSuccess) return e;
    enabled = true;
  }
  if (a.top_k > 1) decode_persistent_kernel<C, MAXKV, true><<<PD_GRID, NT, lds_bytes, s>>>(a);
  else decode_persistent_kernel<C, MAXKV, false><<<PD_GRID, NT, lds_bytes, s>>>(a);
  return hipGetLastError();
}

// A slice of a head holds at most PD_KVBATCH batches of 32 positions in registers. A launch whose last step
// sees more than PD_SHORT_KEYS positions runs the instantiation with twice the slices per head: a compute
// unit streams only ~50 GB/s (32 KB in flight per round trip), and the keys and values of a quarter of a
// long context take an attention workgroup longer to fetch than everything else it does in the layer.
template <int D, int H, bool I8>
hipError_t launch_t(const PersistentArgs& a, hipStream_t s) {
  const int keys = a.pos0 + a.nsteps;  // positions the last step attends to
  if (keys > 32 * PD_KVBATCH * PD_SPLIT_LONG) return hipErrorInvalidValue;
  if (a.short_keys < 0 || a.short_keys > PD_SHORT_KEYS) return hipErrorInvalidValue;
  if (keys <= a.short_keys) return launch_kv<Shape<D, H, I8, PD_SPLIT>, PD_KVBATCH>(a, s);
  return launch_kv<Shape<D, H, I8, PD_SPLIT_LONG>, PD_KVBATCH>(a, s);
}

}  // namespace

PhaseGeom make_geom(int N, int K) {
  PhaseGeom g;
  g.N = N;
  g.cpw = (N + PD_GRID - 1) / PD_GRID;
  g.S = (K + SEG - 1) / SEG;
  return g;
}

size_t slab_float4s(const PhaseGeom& g) { return (size_t)PD_GRID * g.cpw * g.S * 64; }

hipError_t build_slab(const float* W, int ldw, int K, const PhaseGeom& g, const float* rowscale, float4* slab, hipStream_t s) {
  const size_t total = slab_float4s(g);
  build_slab_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(W, ldw, K, g.N, g.cpw, g.S, total, rowscale, slab);
  return hipGetLastError();
}

hipError_t fold_ln_i8(const int32_t* Wq, int ldwq, int K, int N, const float* scale, const float* gamma, const float* beta,
                      const float* bias, float* out_bias, float* gsum, hipStream_t s) {
  fold_ln_i8_kernel<<<(unsigned)((N + 127) / 128), 128, 0, s>>>(Wq, ldwq, K, N, scale, gamma, beta, bias, out_bias, gsum);
  return hipGetLastError();
}

hipError_t fold_ln_bias(const float* W, int ldw, int K, int N, const float* gamma, const float* beta, const float* bias, float* out,
                        float* colsum, hipStream_t s) {
  fold_ln_bias_kernel<<<(unsigned)((N + 127) / 128), 128, 0, s>>>(W, ldw, K, N, gamma, beta, bias, out, colsum);
  return hipGetLastError();
}

hipError_t build_slab_i8(const int32_t* Wq, int ldwq, int K, const PhaseGeom& g, int32_t* slab, hipStream_t s) {
  const size_t total = slab_float4s(g);
  build_slab_i8_kernel<<<(unsigned)((total + 255) / 256), 256, 0, s>>>(Wq, ldwq, K, g.N, g.cpw, g.S, total, slab);
  return hipGetLastError();
}

bool persistent_writes_host_logits(int d, int weight_dtype) { return weight_dtype == 0 && d <= PD_NARROW_D; }

bool persistent_supports(int d, int n_head, int n_ctx, int weight_dtype) {
  if (n_ctx > 32 * PD_KVBATCH * PD_SPLIT_LONG) return false;
  if (weight_dtype == 1) return d == 1600 && n_head == 25;
  return (d == 384 && n_head == 6) || (d == 768 && n_head == 12) || (d == 1024 && n_head == 16) ||
         (d == 1280 && n_head == 20) || (d == 1600 && n_head == 25);
}

hipError_t build_colparams(const float* lparams, int L, int d, int weight_dtype, float* out, hipStream_t s) {
  const size_t n = (size_t)L * PD_GRID * PD_COLP;
  build_colparams_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(lparams, L, d, weight_dtype, make_geom(3 * d, d), make_geom(d, d),
                                                                      make_geom(4 * d, d), make_geom(d, 4 * d), out);
  return hipGetLastError();
}

hipError_t launch_decode_persistent(const PersistentArgs& a, hipStream_t s) {
  if (!persistent_supports(a.d, a.H, a.ctx, a.weight_dtype) || a.top_k < 1 || a.top_k > PD_TOPK) return hipErrorInvalidValue;
#ifdef WGPT_ONLY_D  // experiments: one instantiation, a minute less per build
  if (a.weight_dtype == 0 && a.d == WGPT_ONLY_D) return launch_t<WGPT_ONLY_D, WGPT_ONLY_D / 64, false>(a, s);
#else
  if (a.weight_dtype == 1) return launch_t<1600, 25, true>(a, s);
  switch (a.d) {
    case 384: return launch_t<384, 6, false>(a, s);
    case 768: return launch_t<768, 12, false>(a, s);
    case 1024: return launch_t<1024, 16, false>(a, s);
    case 1280: return launch_t<1280, 20, false>(a, s);
    case 1600: return launch_t<1600, 25, false>(a, s);
  }
#endif
  return hipErrorInvalidValue;
}

}  // namespace wgpt
