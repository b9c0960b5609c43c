// Whole-model entry points: GPT.loadModel (model.js:270-488) becomes
// wgpt_model_create / set_tensor / finalize, GPT.run (model.js:104-268) becomes
// wgpt_prefill (whole window) and wgpt_decode (window extended by one token, served
// from a device-resident KV cache).
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.h"
#include "kernels.h"
#include "model.h"

namespace wgpt {

static std::unordered_map<wgpt_model, Model*>& models() {
  static std::unordered_map<wgpt_model, Model*> m;
  return m;
}
static wgpt_model g_next_model = 1;

static Model* find_model(wgpt_model h) {
  auto it = models().find(h);
  if (it == models().end()) {
    fail(WGPT_ERR_ARG, "unknown model handle %llu", (unsigned long long)h);
    return nullptr;
  }
  return it->second;
}

static int dev_alloc(Model* m, size_t bytes, void** out) {
  void* p = nullptr;
  hipError_t e = hipMalloc(&p, bytes + 16);
  if (e != hipSuccess) return fail(WGPT_ERR_NOMEM, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
  m->allocs.push_back(p);
  *out = p;
  return WGPT_OK;
}

// One named tensor of the weight directory: where it goes and how big it must be.
struct Slot {
  void** dst;
  size_t bytes;
};

static bool parse_name(Model* m, const std::string& name, Slot* slot) {
  const size_t d = m->d, L = m->L;
  const size_t f = sizeof(float);
  if (name == "transformer.wte.weight") { *slot = {(void**)&m->wte, (size_t)m->V * d * f}; return true; }
  if (name == "transformer.wpe.weight") { *slot = {(void**)&m->wpe, (size_t)m->ctx * d * f}; return true; }
  if (name == "transformer.ln_f.weight") { *slot = {(void**)&m->lnf_g, d * f}; return true; }
  if (name == "transformer.ln_f.bias") { *slot = {(void**)&m->lnf_b, d * f}; return true; }
  const char* prefix = "transformer.h.";
  if (name.compare(0, strlen(prefix), prefix) != 0) return false;
  size_t pos = strlen(prefix), end = name.find('.', pos);
  if (end == std::string::npos || end == pos) return false;
  size_t li = 0;
  for (size_t i = pos; i < end; ++i) {
    if (name[i] < '0' || name[i] > '9') return false;
    li = li * 10 + (size_t)(name[i] - '0');
    if (li >= L) return false;
  }
  LayerW& l = m->layers[li];
  const std::string rest = name.substr(end + 1);
  struct Lin { const char* stem; LinW* w; float** bias; size_t K, N; };
  const Lin lins[4] = {{"attn.c_attn", &l.attn, &l.attn_b, d, 3 * d},
                       {"attn.c_proj", &l.proj, &l.proj_b, d, d},
                       {"mlp.c_fc", &l.fc, &l.fc_b, d, 4 * d},
                       {"mlp.c_proj", &l.fc2, &l.fc2_b, 4 * d, d}};
  if (rest == "ln_1.weight") { *slot = {(void**)&l.ln1_g, d * f}; return true; }
  if (rest == "ln_1.bias") { *slot = {(void**)&l.ln1_b, d * f}; return true; }
  if (rest == "ln_2.weight") { *slot = {(void**)&l.ln2_g, d * f}; return true; }
  if (rest == "ln_2.bias") { *slot = {(void**)&l.ln2_b, d * f}; return true; }
  for (const Lin& ln : lins) {
    const std::string stem = ln.stem;
    if (rest == stem + ".bias") { *slot = {(void**)ln.bias, ln.N * f}; return true; }
    if (m->p.weight_dtype == 0) {
      if (rest == stem + ".weight") { *slot = {(void**)&ln.w->w, ln.K * ln.N * f}; return true; }
    } else {
      if (rest == stem + ".weight.q") { *slot = {(void**)&ln.w->q, ln.K * (ln.N / 4) * sizeof(int32_t)}; return true; }
      if (rest == stem + ".weight.scale") { *slot = {(void**)&ln.w->s, ln.N * f}; return true; }
    }
  }
  return false;
}

// C[M,ldc] = epi(A . W + bias) with W fp32 or int8 weight-only.
// With `ln` the LayerNorm that follows in the forward is applied to the finished rows as part of the product.
static int linear(Model* m, int M, int N, int K, const float* A, int lda, const LinW& w, const float* bias, float* C,
                  int ldc, int epi, const float* resid, const LnAfter* ln = nullptr, const KvAfter* kv = nullptr) {
  hipStream_t s = rt().stream;
  hipError_t e;
  bool ln_done = true;
  if (w.q) {
    if (M <= GEMV_MAX_ROWS) {
      e = launch_gemv_kn_i8(M, N, K, A, lda, w.q, N / 4, w.s, bias, C, ldc, epi, resid, m->part, s);
      ln_done = false;
    } else if (M >= 16) {
      e = launch_gemm_i8(M, N, K, A, lda, w.q, N / 4, w.s, bias, C, ldc, epi, resid, m->part, s, ln, kv);
    } else {
      e = launch_dequant_i8(K, N, w.q, N / 4, w.s, m->dq, N, s);
      if (e == hipSuccess) e = launch_gemm(M, N, K, A, lda, m->dq, N, bias, C, ldc, epi, resid, m->part, s, ln, kv);
    }
  } else if (M <= GEMV_MAX_ROWS) {
    e = launch_gemv_kn(M, N, K, A, lda, w.w, N, bias, C, ldc, epi, resid, m->part, s);
    ln_done = false;
  } else {
    e = launch_gemm(M, N, K, A, lda, w.w, N, bias, C, ldc, epi, resid, m->part, s, ln, kv);
  }
  if (e == hipSuccess && !ln_done) {  // the matrix-vector kernels take no follow-ups
    if (kv) e = launch_kv_append(M, kv->d, kv->hs, kv->ctx, kv->pos0, C, kv->Kc, kv->Vc, s);
    if (e == hipSuccess && ln) e = launch_layernorm(M, N, C, ldc, ln->gamma, ln->beta, ln->out, ln->ldo, s);
  }
  if (e != hipSuccess) return fail(WGPT_ERR_HIP, "linear layer launch: %s", hipGetErrorString(e));
  return WGPT_OK;
}

#define LAUNCH(call)                                                                          \
  do {                                                                                        \
    hipError_t e_ = (call);                                                                   \
    if (e_ != hipSuccess) return fail(WGPT_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_));  \
  } while (0)

static int tap(Model* m, int T, size_t index, const float* src) {
  if (!m->taps) return WGPT_OK;
  WGPT_HIP(hipMemcpyAsync(m->taps + index * (size_t)T * m->d, src, sizeof(float) * (size_t)T * m->d,
                          hipMemcpyDeviceToDevice, rt().stream));
  return WGPT_OK;
}

// The forward of model.js:118-240 for T tokens at positions pos0..pos0+T-1, one
// kernel (or two) per instruction block. Token ids are in m->tok_dev.
static int forward_blocks(Model* m, int T, int pos0, bool want_taps) {
  hipStream_t s = rt().stream;
  const int d = m->d, H = m->H, hs = m->hs, hid = 4 * d;
  const float scale = (float)(1.0 / std::sqrt((double)hs));  // model.js:321
  const bool taps = want_taps && m->taps;
  size_t ti = 0;
  int rc;
  LAUNCH(launch_embed(m->tok_dev, T, d, pos0, m->wte, m->wpe, m->x, s));
  if (taps && (rc = tap(m, T, ti, m->x))) return rc;
  ++ti;
  for (int li = 0; li < m->L; ++li) {
    const LayerW& l = m->layers[li];
    float* Kc = m->kv + ((size_t)li * 2 + 0) * m->ctx * d;
    float* Vc = m->kv + ((size_t)li * 2 + 1) * m->ctx * d;
    // without taps the LayerNorm in front of a product is applied by the product before it (see linear)
    if (taps || li == 0) LAUNCH(launch_layernorm(T, d, m->x, d, l.ln1_g, l.ln1_b, m->ln, d, s));
    if (taps && (rc = tap(m, T, ti, m->ln))) return rc;
    ++ti;
    const KvAfter kva = {Kc, Vc, d, hs, m->ctx, pos0};  // the new keys and values join the cache with the product
    if ((rc = linear(m, T, 3 * d, d, m->ln, d, l.attn, l.attn_b, m->qkv, 3 * d, EPI_NONE, nullptr, nullptr, &kva))) return rc;
    LAUNCH(launch_attention(T, pos0, H, hs, scale, m->qkv, 3 * d, Kc, Vc, (size_t)m->ctx * hs, hs, m->att, d, s));
    if (taps) {
      if ((rc = linear(m, T, d, d, m->att, d, l.proj, l.proj_b, m->tmp, d, EPI_NONE, nullptr))) return rc;
      if ((rc = tap(m, T, ti, m->tmp))) return rc;
      LAUNCH(launch_residual((size_t)T * d / 4, m->tmp, m->x, m->x, s));
    } else {
      const LnAfter ln2 = {l.ln2_g, l.ln2_b, m->ln, d};
      if ((rc = linear(m, T, d, d, m->att, d, l.proj, l.proj_b, m->x, d, EPI_RESIDUAL, m->x, &ln2))) return rc;
    }
    ++ti;
    if (taps && (rc = tap(m, T, ti, m->x))) return rc;
    ++ti;
    if (taps) LAUNCH(launch_layernorm(T, d, m->x, d, l.ln2_g, l.ln2_b, m->ln, d, s));
    if (taps && (rc = tap(m, T, ti, m->ln))) return rc;
    ++ti;
    if ((rc = linear(m, T, hid, d, m->ln, d, l.fc, l.fc_b, m->h, hid, EPI_GELU, nullptr))) return rc;
    if (taps) {
      if ((rc = linear(m, T, d, hid, m->h, hid, l.fc2, l.fc2_b, m->tmp, d, EPI_NONE, nullptr))) return rc;
      if ((rc = tap(m, T, ti, m->tmp))) return rc;
      LAUNCH(launch_residual((size_t)T * d / 4, m->tmp, m->x, m->x, s));
    } else {
      if (li + 1 < m->L) {
        const LnAfter ln1 = {m->layers[li + 1].ln1_g, m->layers[li + 1].ln1_b, m->ln, d};
        if ((rc = linear(m, T, d, hid, m->h, hid, l.fc2, l.fc2_b, m->x, d, EPI_RESIDUAL, m->x, &ln1))) return rc;
      } else {
        if ((rc = linear(m, T, d, hid, m->h, hid, l.fc2, l.fc2_b, m->x, d, EPI_RESIDUAL, m->x))) return rc;
      }
    }
    ++ti;
    if (taps && (rc = tap(m, T, ti, m->x))) return rc;
    ++ti;
  }
  if (taps) {
    LAUNCH(launch_layernorm(T, d, m->x, d, m->lnf_g, m->lnf_b, m->ln, d, s));
    if ((rc = tap(m, T, ti, m->ln))) return rc;
    LAUNCH(launch_vocab_gemv(m->V, d, m->ln + (size_t)(T - 1) * d, m->wte, m->logits, s));
  } else {
    // Only the last row is de-embedded (instructions.js:849-856).
    LAUNCH(launch_vocab_gemv_ln(m->V, d, m->x + (size_t)(T - 1) * d, m->lnf_g, m->lnf_b, m->wte, m->logits, nullptr, s));
  }
  return WGPT_OK;
}

// The launches of one decode token at cache position *m->pos_dev (decode mode 0: any model shape): embedding, then
// per layer c_attn (LayerNorm of its input row on the way in, cache append on the way out), attention, c_proj
// (+ residual), c_fc (LayerNorm in, GELU out), mlp c_proj (+ residual); the final LayerNorm with the
// vocabulary projection of that row (instructions.js:849-856), which also advances the position. 5L + 2 launches, none of
// which carries the position as an argument. The products read the decode slabs (a column's K values contiguous).
static int token_launches(Model* m, int pos, bool recording = false) {
  hipStream_t s = rt().stream;
  const int d = m->d, H = m->H, hs = m->hs, hid = 4 * d;
  const float scale = (float)(1.0 / std::sqrt((double)hs));  // model.js:321
  const bool i8 = m->p.weight_dtype == 1;
  const PersistentArgs& a = m->pa;
  const LayerParamOffsets po = layer_param_offsets(d);
  const size_t lane_bytes = i8 ? sizeof(int32_t) : sizeof(float4);
  // fp32 slabs carry the LayerNorm gains and their biases the LayerNorm biases: the row is only normalised
  const int ln_mode = i8 ? GEMV_ROW_LAYERNORM : GEMV_ROW_NORMALISE;
  // `pos` is what the host knows of the token's cache position (0 when the launches are recorded for replay); the
  // launches themselves read it from the device. It is only a hint to the attention: the slices of the cache up to it
  // request their rows before they have read the position, the others look first.
  const bool sliced = m->att_nslice > 1;  // a cache of one slice is served by the one-workgroup-per-head kernel
  LAUNCH(launch_embed_at(m->tok_dev, d, m->pos_dev, m->wte, m->wpe, m->x, s));
  for (int li = 0; li < m->L; ++li) {
    const LayerW& l = m->layers[li];
    float* Kc = m->kv + ((size_t)li * 2 + 0) * m->ctx * d;
    float* Vc = m->kv + ((size_t)li * 2 + 1) * m->ctx * d;
    const KvAfter kva = {Kc, Vc, d, hs, m->ctx, 0};
    const char* slab = static_cast<const char*>(a.slabs) + (size_t)li * a.slab_stride * lane_bytes;
    const float* lp = a.lparams + (size_t)li * po.stride;
    LAUNCH(launch_gemv_slab(3 * d, d, slab, i8, lp + po.sA, m->x, ln_mode, l.ln1_g, l.ln1_b, lp + po.bA, m->qkv, EPI_NONE, nullptr, &kva,
                            m->pos_dev, s));
    if (sliced) {  // a workgroup per (head, slice of the cache), merged as c_proj stages its row
      // (a recorded token merges all slices: those beyond the context hold zeros with weight zero)
      const int per = attention_decode_slice_positions(hs);
      const AttnSlices sl = {m->att_part, m->att_nslice, hs, recording ? m->att_nslice : std::min(m->att_nslice, pos / per + 1)};
      LAUNCH(launch_attention_decode_slices(H, hs, m->ctx, scale, m->qkv, Kc, Vc, &sl, m->pos_dev, pos, s));
      LAUNCH(launch_gemv_slab(d, d, slab + a.slab_offC * lane_bytes, i8, lp + po.sC, nullptr, GEMV_ROW_PLAIN, nullptr, nullptr, lp + po.bC, m->x,
                              EPI_RESIDUAL, m->x, nullptr, m->pos_dev, s, &sl));
    } else {
      LAUNCH(launch_attention_decode(H, hs, m->ctx, scale, m->qkv, Kc, Vc, m->att, m->pos_dev, s));
      LAUNCH(launch_gemv_slab(d, d, slab + a.slab_offC * lane_bytes, i8, lp + po.sC, m->att, GEMV_ROW_PLAIN, nullptr, nullptr, lp + po.bC, m->x,
                              EPI_RESIDUAL, m->x, nullptr, m->pos_dev, s));
    }
    LAUNCH(launch_gemv_slab(hid, d, slab + a.slab_offD * lane_bytes, i8, lp + po.sD, m->x, ln_mode, l.ln2_g, l.ln2_b, lp + po.bD, m->h, EPI_GELU,
                            nullptr, nullptr, m->pos_dev, s));
    LAUNCH(launch_gemv_slab(d, hid, slab + a.slab_offE * lane_bytes, i8, lp + po.sE, m->h, GEMV_ROW_PLAIN, nullptr, nullptr, lp + po.bE, m->x,
                            EPI_RESIDUAL, m->x, nullptr, m->pos_dev, s));
  }
  LAUNCH(launch_vocab_gemv_ln(m->V, d, m->x, m->lnf_g, m->lnf_b, m->wte, m->logits, m->pos_dev, s));
  return WGPT_OK;
}

// Sends the host's cache position to pos_dev (the start of a decode call of mode 0; the token launches advance it).
static int upload_position(Model* m) {
  m->pin[2] = m->pos;  // every earlier use of the word has completed: each call ends with a synchronisation
  WGPT_HIP(hipMemcpyAsync(m->pos_dev, &m->pin[2], sizeof(int), hipMemcpyHostToDevice, rt().stream));
  return WGPT_OK;
}

// One decode token of mode 0 at the position in pos_dev. Because no launch carries the position, the token's launches
// can be recorded once as a HIP graph (kernel nodes only) and replayed: WEBGPT_AMD_TOKEN_GRAPH=1 does that. It is
// not the default: on MI355X the replay is exactly as fast as issuing the launches (117M: 0.4338 against 0.4326
// ms/token; a token is bound by its 5L + 2 dependent kernels of 4-7 us each, not by the host), and rocprofv3 crashed
// in its own graph handling on the 242-node graph of a 48-layer model.
static int decode_token_blocks(Model* m, int pos) {
  hipStream_t s = rt().stream;
  if (!m->slabs_ok) return fail(WGPT_ERR_STATE, "decode: the decode layouts of the model were not built");
  if (!m->token_graph_tried) {
    m->token_graph_tried = true;
    const char* on = getenv("WEBGPT_AMD_TOKEN_GRAPH");
    if (on && on[0] == '1') {
      WGPT_HIP(hipStreamSynchronize(s));
      // a recording run changes nothing on the device: what is recorded is replayed below
      if (hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal) == hipSuccess) {
        const int rc = token_launches(m, 0, true);
        hipGraph_t g = nullptr;
        const hipError_t e = hipStreamEndCapture(s, &g);
        if (rc == WGPT_OK && e == hipSuccess && g && hipGraphInstantiate(&m->token_graph_exec, g, nullptr, nullptr, 0) == hipSuccess) {
          m->token_graph = g;
        } else {
          if (g) (void)hipGraphDestroy(g);
          m->token_graph_exec = nullptr;
          (void)hipGetLastError();
        }
      } else {
        (void)hipGetLastError();
      }
    }
  }
  if (m->token_graph_exec) {
    WGPT_HIP(hipGraphLaunch(m->token_graph_exec, s));
    return WGPT_OK;
  }
  return token_launches(m, pos);
}

// Prepares the decode paths: slab-layout copies of the linear weights and the per-layer parameter blocks
// (any shape), then, for the shapes the persistent whole-token kernel is built for, its per-workgroup
// parameter blocks and exchange buffers. Leaves m->persist_ok false (and the per-block path in charge) for
// shapes the persistent kernel does not cover.
static int setup_persistent(Model* m) {
  m->persist_ok = false;
  const int d = m->d, hid = 4 * d, G = PD_GRID, split = PD_SPLIT_LONG;  // (the exchange buffer of the larger split)
  const bool i8 = m->p.weight_dtype == 1;
  PersistentArgs& a = m->pa;
  a = PersistentArgs{};
  a.L = m->L; a.H = m->H; a.d = d; a.ctx = m->ctx; a.V = m->V;
  a.weight_dtype = m->p.weight_dtype;
  a.scale = (float)(1.0 / std::sqrt((double)m->hs));
  const PhaseGeom gA = make_geom(3 * d, d), gC = make_geom(d, d), gD = make_geom(hid, d), gE = make_geom(d, hid);
  a.rows_per_wg = (m->V + G - 1) / G;
  const int attw = m->H * split * (m->hs + 2);

  int rc;
  // all slabs in one allocation, all small per-layer parameters in another
  a.slab_offC = slab_float4s(gA);
  a.slab_offD = a.slab_offC + slab_float4s(gC);
  a.slab_offE = a.slab_offD + slab_float4s(gD);
  a.slab_stride = a.slab_offE + slab_float4s(gE);
  // an item lane is a float4 (fp32) or one word of four int8 (int8)
  const size_t lane_bytes = i8 ? sizeof(int32_t) : sizeof(float4);
  char* slabs;
  if ((rc = dev_alloc(m, a.slab_stride * (size_t)m->L * lane_bytes, (void**)&slabs))) return rc;
  const LayerParamOffsets po = layer_param_offsets(d);
  float* lparams;
  if ((rc = dev_alloc(m, sizeof(float) * (size_t)po.stride * m->L, (void**)&lparams))) return rc;
  for (int i = 0; i < m->L; ++i) {
    const LayerW& l = m->layers[i];
    char* slb = slabs + (size_t)i * a.slab_stride * lane_bytes;
    if (i8) {
      int32_t* sl = (int32_t*)slb;
      LAUNCH(build_slab_i8(l.attn.q, 3 * d / 4, d, gA, sl, rt().stream));
      LAUNCH(build_slab_i8(l.proj.q, d / 4, d, gC, sl + a.slab_offC, rt().stream));
      LAUNCH(build_slab_i8(l.fc.q, hid / 4, d, gD, sl + a.slab_offD, rt().stream));
      LAUNCH(build_slab_i8(l.fc2.q, d / 4, hid, gE, sl + a.slab_offE, rt().stream));
    } else {
      float4* sl = (float4*)slb;
      // the two LayerNorms go into the matrices they feed: diag(gamma) W here, beta W into the bias below
      LAUNCH(build_slab(l.attn.w, 3 * d, d, gA, l.ln1_g, sl, rt().stream));
      LAUNCH(build_slab(l.proj.w, d, d, gC, nullptr, sl + a.slab_offC, rt().stream));
      LAUNCH(build_slab(l.fc.w, hid, d, gD, l.ln2_g, sl + a.slab_offD, rt().stream));
      LAUNCH(build_slab(l.fc2.w, d, hid, gE, nullptr, sl + a.slab_offE, rt().stream));
    }
    float* lp = lparams + (size_t)i * po.stride;
    const struct { int off; const float* src; int n; } parts[12] = {
        {po.bA, l.attn_b, 3 * d}, {po.bC, l.proj_b, d}, {po.bD, l.fc_b, hid}, {po.bE, l.fc2_b, d},
        {po.ln1g, l.ln1_g, d},    {po.ln1b, l.ln1_b, d}, {po.ln2g, l.ln2_g, d}, {po.ln2b, l.ln2_b, d},
        {po.sA, l.attn.s, 3 * d}, {po.sC, l.proj.s, d}, {po.sD, l.fc.s, hid}, {po.sE, l.fc2.s, d}};
    for (const auto& pt : parts)
      if (pt.src) WGPT_HIP(hipMemcpyAsync(lp + pt.off, pt.src, sizeof(float) * pt.n, hipMemcpyDeviceToDevice, rt().stream));
    if (!i8) {
      LAUNCH(fold_ln_bias(l.attn.w, 3 * d, d, 3 * d, l.ln1_g, l.ln1_b, l.attn_b, lp + po.bA, lp + po.sA, rt().stream));
      LAUNCH(fold_ln_bias(l.fc.w, hid, d, hid, l.ln2_g, l.ln2_b, l.fc_b, lp + po.bD, lp + po.sD, rt().stream));
    } else {
      // (the plain biases stay where they are: the one-launch-per-block path applies the LayerNorm itself)
      LAUNCH(fold_ln_i8(l.attn.q, 3 * d / 4, d, 3 * d, l.attn.s, l.ln1_g, l.ln1_b, l.attn_b, lp + po.fA, lp + po.gA, rt().stream));
      LAUNCH(fold_ln_i8(l.fc.q, hid / 4, d, hid, l.fc.s, l.ln2_g, l.ln2_b, l.fc_b, lp + po.fD, lp + po.gD, rt().stream));
    }
  }
  a.slabs = slabs;
  a.lparams = lparams;
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  m->slabs_ok = true;
  // The slabs and the folded parameters serve both decode paths (the one-launch-per-block path reads a column of a
  // slab as one contiguous run of K); what follows is for the persistent kernel and the shapes it is built for.
  if (m->hs != 64) return WGPT_OK;
  if (rt().compute_units < G) return WGPT_OK;
  if (!persistent_supports(d, m->H, m->ctx, m->p.weight_dtype)) return WGPT_OK;
  float* colparams;
  if ((rc = dev_alloc(m, sizeof(float) * (size_t)m->L * PD_GRID * PD_COLP, (void**)&colparams))) return rc;
  LAUNCH(build_colparams(lparams, m->L, d, i8 ? 1 : 0, colparams, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  a.slabs = slabs;
  a.lparams = lparams;
  a.colparams = colparams;
  a.wte = m->wte; a.wpe = m->wpe; a.lnf_g = m->lnf_g; a.lnf_b = m->lnf_b;
  a.kv = m->kv;
  const size_t words = (size_t)3 * d + attw + d + hid + d + 2 * PD_TOPK * G;
  unsigned long long* buf;
  if ((rc = dev_alloc(m, words * sizeof(unsigned long long), (void**)&buf))) return rc;
  WGPT_HIP(hipMemsetAsync(buf, 0, words * sizeof(unsigned long long), rt().stream));
  a.bufQKV = buf;
  a.bufATT = a.bufQKV + 3 * d;
  a.bufR1 = a.bufATT + attw;
  a.bufH = a.bufR1 + d;
  a.bufR2 = a.bufH + hid;
  a.bufAM = a.bufR2 + d;
  m->perr = reinterpret_cast<int*>(m->logits + m->V);
  WGPT_HIP(hipMemsetAsync(m->perr, 0, sizeof(int), rt().stream));
  a.logits = m->logits;
  a.tok = m->tok_dev;
  a.out_tok = m->out_tok_dev;
  a.err = m->perr;
  {
    // measured optima on MI355X (coordinate descent on ms/token at contexts of 130-770; the
    // curves are flat within a few percent around them and over context length);
    // wgpt_model_tune_poll_delays searches around them on the GPU at hand,
    // WEBGPT_AMD_POLL_DELAYS="a,b,c,d,e,f,g" overrides them for experiments
    static const int tuned[5][7] = {{16, 4, 22, 78, 24, 28, 48},    // d <= 768
                                    {36, 0, 26, 82, 40, 40, 4},     // d = 1024
                                    {20, 0, 34, 100, 16, 16, 52},   // d = 1280
                                    {8, 12, 22, 84, 20, 12, 44},    // d = 1600, int8
                                    {32, 0, 48, 96, 4, 20, 40}};    // d = 1600, fp32
    // growth of [2] and [3] per 1024 positions of context (the best values at contexts of 100, 350, 650 and 900
    // positions lie on a line: 117M 80, 88, 88, 104 for [3]; int8 88, 104, 128, 136)
    static const int slopes[5][2] = {{11, 28}, {0, 46}, {9, 70}, {20, 61}, {0, 0}};
    const int row = d <= 768 ? 0 : d == 1024 ? 1 : d == 1280 ? 2 : i8 ? 3 : 4;
    const int* dflt = tuned[row];
    for (int i = 0; i < 7; ++i) a.delay[i] = dflt[i];
    a.att_slope[0] = slopes[row][0];
    a.att_slope[1] = slopes[row][1];
    if (const char* e = getenv("WEBGPT_AMD_POLL_DELAYS")) {
      int v[7];
      if (sscanf(e, "%d,%d,%d,%d,%d,%d,%d", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5], &v[6]) == 7)
        for (int i = 0; i < 7; ++i) a.delay[i] = v[i] < 0 ? 0 : (v[i] > 1024 ? 1024 : v[i]);
    }
    if (const char* e = getenv("WEBGPT_AMD_POLL_SLOPES")) {
      int v[2];
      if (sscanf(e, "%d,%d", &v[0], &v[1]) == 2)
        for (int i = 0; i < 2; ++i) a.att_slope[i] = v[i] < 0 ? 0 : (v[i] > 1024 ? 1024 : v[i]);
    }
  }
  // a wait that takes this many poll rounds (a quarter of a second) means a workgroup is not running;
  // WEBGPT_AMD_SPIN_LIMIT lowers it (tests of the fallback force an expiry this way: with 0 a wait
  // gives up when its first look finds a word missing, which without poll delays is certain)
  a.spin_limit = 1u << 18;
  if (const char* e = getenv("WEBGPT_AMD_SPIN_LIMIT")) {
    char* end = nullptr;
    const long v = strtol(e, &end, 10);
    if (end != e && v >= 0 && v < (1l << 30)) a.spin_limit = (unsigned)v;
  }
  // context length from which a launch uses twice the attention slices per head (WEBGPT_AMD_SHORT_KEYS for tuning)
  a.short_keys = PD_SHORT_KEYS;
  if (const char* e = getenv("WEBGPT_AMD_SHORT_KEYS")) {
    char* end = nullptr;
    const long v = strtol(e, &end, 10);
    if (end != e && v >= 0 && v <= PD_SHORT_KEYS) a.short_keys = (int)v;
  }
  a.trace = nullptr;
#ifdef WGPT_TRACE
  // Profiling builds: per-workgroup clock samples of the last step of each launch.
  if ((rc = dev_alloc(m, sizeof(unsigned long long) * 512 * G, (void**)&a.trace))) return rc;
  WGPT_HIP(hipMemsetAsync(a.trace, 0, sizeof(unsigned long long) * 512 * G, rt().stream));
#endif
  m->epoch = 0;
  // WEBGPT_AMD_EPOCH_START: tests start the counter just below its limit to run the restart above
  if (const char* e = getenv("WEBGPT_AMD_EPOCH_START")) {
    char* end = nullptr;
    const unsigned long v = strtoul(e, &end, 10);
    if (end != e && v <= 0x7fffffffu) m->epoch = (unsigned)v;
  }
  m->persist_ok = true;
  return WGPT_OK;
}

// Runs `steps` greedy decode steps from position m->pos with the persistent kernel.
// The first token is in m->tok_dev[0]; chosen ids land in m->out_tok_dev.
// top_k == 1: greedy. Otherwise u_dev holds the steps' uniform draws.
// host_results: the call ends with a read-back (finish_timed, finish_steps): the kernel then reports its error word, and
// where the shape allows the last step's logits, in pinned host memory itself instead of through copies behind it.
static int decode_persistent(Model* m, int steps, int top_k = 1, double temperature = 1.0, const double* u_dev = nullptr, int token = -1,
                             bool host_results = false) {
  PersistentArgs a = m->pa;
  a.host_logits = nullptr;
  a.host_done = nullptr;
  if (token >= 0) {  // the first token travels with the launch instead of through tok_dev
    a.tok = nullptr;
    a.tok_value = token;
  }
  a.top_k = top_k;
  a.temperature = temperature;
  a.u = u_dev;
  const unsigned per_step = persistent_epochs_per_step(m->L);
  if (m->epoch > 0x7fffffffu - per_step * (unsigned)steps - 8u) {
    // epoch counter about to leave the positive ints (the kernel's error word is the epoch of the wait that
    // expired, as an int; negative values are its other codes): start over from clean exchange buffers
    const size_t words = (size_t)(a.bufAM + 2 * PD_TOPK * PD_GRID - a.bufQKV);
    WGPT_HIP(hipMemsetAsync(a.bufQKV, 0, words * sizeof(unsigned long long), rt().stream));
    m->epoch = 0;
  }
  a.ebase = m->epoch;
  a.pos0 = m->pos;
  a.nsteps = steps;
  // steps that attend to at most PD_SHORT_KEYS positions run the instantiation with half the key/value
  // registers; a run that crosses that context length is two launches, the second taking its first
  // token from the ids the first one wrote
  const int short_steps = a.short_keys - m->pos;
  if (short_steps > 0 && short_steps < steps) {
    a.nsteps = short_steps;
    LAUNCH(launch_decode_persistent(a, rt().stream));
    a.ebase += per_step * (unsigned)short_steps;
    a.pos0 += short_steps;
    a.tok = a.out_tok + short_steps - 1;
    a.out_tok += short_steps;
    if (a.u) a.u += short_steps;
    a.nsteps = steps - short_steps;
  }
  if (host_results) {  // (the last launch of the call only)
    m->pin[1] = -1;  // every earlier use of the word has completed: each call ends with a synchronisation
    a.host_done = &m->pin[1];
    if (persistent_writes_host_logits(m->d, m->p.weight_dtype) && a.rows_per_wg <= 4 * m->d) a.host_logits = m->logits_pin;
  }
  LAUNCH(launch_decode_persistent(a, rt().stream));
  m->res_host_done = a.host_done != nullptr;
  m->res_host_logits = a.host_logits != nullptr;
  m->epoch += per_step * (unsigned)steps;
  return WGPT_OK;
}

// After the stream has drained: did a bounded wait of the persistent kernel expire?
static int check_persistent(Model* m) {
#ifdef WGPT_TRACE
  if (const char* path = getenv("WGPT_TRACE_FILE")) {
    std::vector<unsigned long long> h(512 * (size_t)PD_GRID);
    WGPT_HIP(hipMemcpy(h.data(), m->pa.trace, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    if (FILE* f = fopen(path, "wb")) {
      fwrite(h.data(), sizeof(unsigned long long), h.size(), f);
      fclose(f);
    }
  }
#endif
  // the error word came back with the call's results (read_back)
  const int herr = m->pin[1];
  if (herr != 0) {
    (void)hipMemset(m->perr, 0, sizeof(int));
    m->persist_ok = false;  // do not trust the exchange buffers again
    m->decode_mode = 0;
    if (herr == -16)
      return fail(WGPT_ERR_DEVICE, "persistent decode kernel: its LDS rows are not 16-byte aligned (build problem); the persistent path is now disabled");
    if (herr == -1)
      return fail(WGPT_ERR_DEVICE, "persistent decode kernel: the launch did not run to its end; the persistent path is now disabled");
    return fail(WGPT_ERR_DEVICE, "persistent decode kernel: a bounded wait expired at epoch %d; the persistent path is now disabled", herr);
  }
  return WGPT_OK;
}

// Brings the error word and, if asked for, the logits of the call to the host and drains the stream. The logits cross
// the bus into pinned memory (a copy into the caller's pageable buffer is staged by the runtime in pieces) and are
// handed over with a host copy; the error word rides behind them. What a persistent launch has written into pinned
// memory itself (res_host_done, res_host_logits) is not copied again.
static int read_back(Model* m, float* logits) {
  const bool host_done = m->res_host_done, host_logits = m->res_host_logits;
  m->res_host_done = m->res_host_logits = false;
  const bool copy_logits = logits && !host_logits, copy_err = m->perr && !host_done;
  if (copy_logits && copy_err) {
    WGPT_HIP(hipMemcpyAsync(m->logits_pin, m->logits, sizeof(float) * ((size_t)m->V + 1), hipMemcpyDeviceToHost, rt().stream));
  } else {
    if (copy_logits) WGPT_HIP(hipMemcpyAsync(m->logits_pin, m->logits, sizeof(float) * (size_t)m->V, hipMemcpyDeviceToHost, rt().stream));
    if (copy_err) WGPT_HIP(hipMemcpyAsync(&m->pin[1], m->perr, sizeof(int), hipMemcpyDeviceToHost, rt().stream));
  }
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  if (copy_logits && copy_err) memcpy(&m->pin[1], m->logits_pin + m->V, sizeof(int));
  if (host_done && m->pin[1] == -1) {
    // the kernel did not reach its end: a wait has expired and the device's word says which
    WGPT_HIP(hipMemcpy(&m->pin[1], m->perr, sizeof(int), hipMemcpyDeviceToHost));
    if (m->pin[1] == 0) m->pin[1] = -1;
  }
  if (logits) memcpy(logits, m->logits_pin, sizeof(float) * (size_t)m->V);
  return WGPT_OK;
}

static int finish_timed(Model* m, float* logits) {
  WGPT_HIP(hipEventRecord(m->ev1, rt().stream));
  const int rc = read_back(m, logits);
  if (rc) return rc;
  WGPT_HIP(hipEventElapsedTime(&m->last_ms, m->ev0, m->ev1));
  return WGPT_OK;
}

// The ids of a multi-step call come back through pinned memory as well: a copy into the caller's pageable array is
// staged by the runtime and costs tens of microseconds per call. Ends with the stream drained.
static int finish_steps(Model* m, int32_t* out_tokens, const int32_t* ids_dev, int steps, float* logits) {
  WGPT_HIP(hipEventRecord(m->ev1, rt().stream));
  WGPT_HIP(hipMemcpyAsync(m->ids_pin, ids_dev, sizeof(int32_t) * (size_t)steps, hipMemcpyDeviceToHost, rt().stream));
  const int rc = read_back(m, logits);
  if (rc) return rc;
  memcpy(out_tokens, m->ids_pin, sizeof(int32_t) * (size_t)steps);
  WGPT_HIP(hipEventElapsedTime(&m->last_ms, m->ev0, m->ev1));
  return WGPT_OK;
}

static void destroy_model(Model* m) {
  if (m->token_graph_exec) (void)hipGraphExecDestroy(m->token_graph_exec);
  if (m->token_graph) (void)hipGraphDestroy(m->token_graph);
  for (void* p : m->allocs) (void)hipFree(p);
  if (m->pin) (void)hipHostFree(m->pin);
  if (m->logits_pin) (void)hipHostFree(m->logits_pin);
  if (m->ids_pin) (void)hipHostFree(m->ids_pin);
  if (m->ev0) (void)hipEventDestroy(m->ev0);
  if (m->ev1) (void)hipEventDestroy(m->ev1);
  delete m;
}

void destroy_all_models() {
  for (auto& kv : models()) destroy_model(kv.second);
  models().clear();
}

}  // namespace wgpt

using namespace wgpt;

extern "C" {

int wgpt_model_create(const wgpt_params* p, wgpt_model* out) {
  WGPT_REQUIRE_INIT();
  if (!p || !out) return fail(WGPT_ERR_ARG, "wgpt_model_create: NULL argument");
  if (p->n_layer < 1 || p->n_head < 1 || p->n_embd < 1 || p->n_ctx < 1 || p->vocab_size < 1)
    return fail(WGPT_ERR_ARG, "wgpt_model_create: all of n_layer, n_head, n_embd, n_ctx, vocab_size must be positive");
  // model.js:294-297
  if (p->n_embd % 4 != 0) return fail(WGPT_ERR_ARG, "Model load failed: n_embd must be divisible by 4.");
  if (p->n_embd % p->n_head != 0) return fail(WGPT_ERR_ARG, "Model load failed: n_embd must be divisible by n_head.");
  if ((p->n_embd / p->n_head) % 4 != 0) return fail(WGPT_ERR_ARG, "Model load failed: n_embd / n_head must be divisible by 4.");
  if (p->n_embd % 8 != 0) return fail(WGPT_ERR_ARG, "Cols must be divisible by 16.");  // FastMatMul on [*, n_embd]
  if (p->n_embd / p->n_head > 256) return fail(WGPT_ERR_ARG, "wgpt_model_create: head size above 256 is not supported");
  // the decode kernels stage an input row of up to 4 n_embd floats in 48 KB of LDS
  if (p->n_embd > 3072) return fail(WGPT_ERR_ARG, "wgpt_model_create: n_embd above 3072 is not supported");
  if (p->n_ctx > 12288) return fail(WGPT_ERR_ARG, "wgpt_model_create: n_ctx above 12288 is not supported");
  if (p->weight_dtype != 0 && p->weight_dtype != 1) return fail(WGPT_ERR_ARG, "wgpt_model_create: weight_dtype must be 0 (fp32) or 1 (int8)");
  if (p->max_prefill < 0 || p->max_prefill > p->n_ctx) return fail(WGPT_ERR_ARG, "wgpt_model_create: max_prefill must be in [0, n_ctx]");
  Model* m = new Model();
  m->p = *p;
  m->L = p->n_layer; m->H = p->n_head; m->d = p->n_embd; m->ctx = p->n_ctx; m->V = p->vocab_size;
  m->hs = m->d / m->H;
  m->maxT = p->max_prefill ? p->max_prefill : p->n_ctx;
  m->layers.resize(m->L);
  *out = g_next_model++;
  models()[*out] = m;
  return WGPT_OK;
}

int wgpt_model_set_tensor(wgpt_model h, const char* name, const void* data, size_t bytes) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (m->finalized) return fail(WGPT_ERR_STATE, "wgpt_model_set_tensor: model already finalised");
  if (!name || !data) return fail(WGPT_ERR_ARG, "wgpt_model_set_tensor: NULL argument");
  Slot slot;
  if (!parse_name(m, name, &slot)) return fail(WGPT_ERR_ARG, "wgpt_model_set_tensor: unknown tensor name '%s'", name);
  if (bytes != slot.bytes) return fail(WGPT_ERR_ARG, "wgpt_model_set_tensor: '%s' needs %zu bytes, got %zu", name, slot.bytes, bytes);
  if (!*slot.dst) {
    int rc = dev_alloc(m, bytes, slot.dst);
    if (rc) return rc;
  }
  WGPT_HIP(hipMemcpyAsync(*slot.dst, data, bytes, hipMemcpyHostToDevice, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  return WGPT_OK;
}

int wgpt_model_finalize(wgpt_model h) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (m->finalized) return WGPT_OK;
  const bool i8 = m->p.weight_dtype == 1;
  if (!m->wte || !m->wpe || !m->lnf_g || !m->lnf_b) return fail(WGPT_ERR_STATE, "wgpt_model_finalize: embeddings or final layer norm missing");
  for (int i = 0; i < m->L; ++i) {
    const LayerW& l = m->layers[i];
    const LinW* lw[4] = {&l.attn, &l.proj, &l.fc, &l.fc2};
    bool ok = l.ln1_g && l.ln1_b && l.ln2_g && l.ln2_b && l.attn_b && l.proj_b && l.fc_b && l.fc2_b;
    for (const LinW* w : lw) ok = ok && (i8 ? (w->q && w->s) : (w->w != nullptr));
    if (!ok) return fail(WGPT_ERR_STATE, "wgpt_model_finalize: layer %d is missing tensors", i);
  }
  const size_t d = m->d, T = m->maxT, f = sizeof(float);
  int rc;
  if ((rc = dev_alloc(m, (size_t)m->L * 2 * m->ctx * d * f, (void**)&m->kv))) return rc;
  if ((rc = dev_alloc(m, T * d * f, (void**)&m->x))) return rc;
  if ((rc = dev_alloc(m, T * d * f, (void**)&m->ln))) return rc;
  if ((rc = dev_alloc(m, T * 3 * d * f, (void**)&m->qkv))) return rc;
  if ((rc = dev_alloc(m, T * d * f, (void**)&m->att))) return rc;
  if ((rc = dev_alloc(m, T * d * f, (void**)&m->tmp))) return rc;
  if ((rc = dev_alloc(m, T * 4 * d * f, (void**)&m->h))) return rc;
  // the error word of the persistent kernel lives right behind the logits, so that one copy brings both back
  if ((rc = dev_alloc(m, ((size_t)m->V + 1) * f, (void**)&m->logits))) return rc;
  if ((rc = dev_alloc(m, T * sizeof(int32_t), (void**)&m->tok_dev))) return rc;
  if (!m->pin) {
    WGPT_HIP(hipHostMalloc((void**)&m->pin, 4 * sizeof(int32_t), hipHostMallocDefault));
    m->pin[0] = m->pin[1] = m->pin[2] = m->pin[3] = 0;
    WGPT_HIP(hipHostMalloc((void**)&m->logits_pin, sizeof(float) * ((size_t)m->V + 1), hipHostMallocDefault));
    WGPT_HIP(hipHostMalloc((void**)&m->ids_pin, sizeof(int32_t) * (size_t)m->ctx, hipHostMallocDefault));
  }
  if ((rc = dev_alloc(m, sizeof(int), (void**)&m->pos_dev))) return rc;
  m->att_nslice = attention_decode_slices(m->hs, m->ctx);
  if (m->att_nslice > 1 && (rc = dev_alloc(m, (size_t)m->H * m->att_nslice * (m->hs + 4) * f, (void**)&m->att_part))) return rc;
  WGPT_HIP(hipMemsetAsync(m->pos_dev, 0, sizeof(int), rt().stream));
  if ((rc = dev_alloc(m, (size_t)m->ctx * sizeof(int32_t), (void**)&m->out_tok_dev))) return rc;
  if ((rc = dev_alloc(m, (size_t)m->ctx * sizeof(int32_t), (void**)&m->out_samp_dev))) return rc;
  if ((rc = dev_alloc(m, (size_t)m->ctx * sizeof(double), (void**)&m->u_dev))) return rc;
  size_t ws = gemv_workspace_floats(GEMV_MAX_ROWS, 4 * (int)d, (int)d);
  const size_t ws2 = gemv_workspace_floats(GEMV_MAX_ROWS, (int)d, 4 * (int)d);
  if (ws2 > ws) ws = ws2;
  const size_t ws3 = gemm_workspace_floats((int)T, 4 * (int)d);  // split-K partial sums of the prefill GEMMs
  if (ws3 > ws) ws = ws3;
  if ((rc = dev_alloc(m, ws * f, (void**)&m->part))) return rc;
  if (i8 && (rc = dev_alloc(m, d * 4 * d * f, (void**)&m->dq))) return rc;
  if ((m->p.flags & WGPT_FLAG_TAPS) && (rc = dev_alloc(m, (size_t)(2 + 6 * m->L) * T * d * f, (void**)&m->taps))) return rc;
  WGPT_HIP(hipMemsetAsync(m->kv, 0, (size_t)m->L * 2 * m->ctx * d * f, rt().stream));
  WGPT_HIP(hipEventCreate(&m->ev0));
  WGPT_HIP(hipEventCreate(&m->ev1));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  if ((rc = setup_persistent(m))) return rc;
  m->decode_mode = m->persist_ok ? 1 : 0;
  m->pos = 0;
  m->finalized = true;
  if ((m->p.flags & WGPT_FLAG_TUNE_DELAYS) && m->persist_ok) return wgpt_model_tune_poll_delays(h, 2, nullptr, nullptr, nullptr);
  return WGPT_OK;
}

int wgpt_prefill(wgpt_model h, const int32_t* tokens, int T, float* logits) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  m->res_host_done = m->res_host_logits = false;  // (left set by a call that failed between its launch and its read-back)
  if (!m->finalized) return fail(WGPT_ERR_STATE, "wgpt_prefill: model not finalised");
  if (!tokens || T < 1) return fail(WGPT_ERR_ARG, "wgpt_prefill: tokens and T >= 1 required");
  if (T > m->maxT) return fail(WGPT_ERR_ARG, "wgpt_prefill: T = %d exceeds max_prefill = %d", T, m->maxT);
  for (int i = 0; i < T; ++i)
    if (tokens[i] < 0 || tokens[i] >= m->V) return fail(WGPT_ERR_ARG, "wgpt_prefill: token id %d at %d outside [0, %d)", tokens[i], i, m->V);
  WGPT_HIP(hipMemcpyAsync(m->tok_dev, tokens, sizeof(int32_t) * (size_t)T, hipMemcpyHostToDevice, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  WGPT_HIP(hipEventRecord(m->ev0, rt().stream));
  m->pos = 0;
  m->tap_T = 0;
  m->x_rows = 0;
  int rc = forward_blocks(m, T, 0, true);
  if (rc) return rc;
  rc = finish_timed(m, logits);
  if (rc) return rc;
  m->pos = T;
  m->tap_T = m->taps ? T : 0;
  m->x_rows = T;
  return WGPT_OK;
}

int wgpt_decode(wgpt_model h, int32_t token, float* logits) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  m->res_host_done = m->res_host_logits = false;  // (left set by a call that failed between its launch and its read-back)
  m->x_rows = 0;
  if (!m->finalized) return fail(WGPT_ERR_STATE, "wgpt_decode: model not finalised");
  if (token < 0 || token >= m->V) return fail(WGPT_ERR_ARG, "wgpt_decode: token id %d outside [0, %d)", token, m->V);
  if (m->pos >= m->ctx) return fail(WGPT_ERR_STATE, "wgpt_decode: context of %d positions is full; prefill a slid window", m->ctx);
  int rc;
  if (m->decode_mode != 1) {  // (the persistent kernel takes the token as a launch argument)
    m->pin[0] = token;  // every earlier use of the word has completed: each call ends with a synchronisation
    WGPT_HIP(hipMemcpyAsync(m->tok_dev, &m->pin[0], sizeof(int32_t), hipMemcpyHostToDevice, rt().stream));
    if ((rc = upload_position(m))) return rc;
  }
  WGPT_HIP(hipEventRecord(m->ev0, rt().stream));
  rc = m->decode_mode == 1 ? decode_persistent(m, 1, 1, 1.0, nullptr, token, true) : decode_token_blocks(m, m->pos);
  if (rc) return rc;
  rc = finish_timed(m, logits);
  if (rc) return rc;
  if (m->decode_mode == 1 && (rc = check_persistent(m))) return rc;
  m->pos += 1;
  return WGPT_OK;
}

int wgpt_decode_greedy(wgpt_model h, int32_t token, int steps, int32_t* out_tokens, float* logits) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  m->res_host_done = m->res_host_logits = false;  // (left set by a call that failed between its launch and its read-back)
  m->x_rows = 0;
  if (!m->finalized) return fail(WGPT_ERR_STATE, "wgpt_decode_greedy: model not finalised");
  if (token < 0 || token >= m->V) return fail(WGPT_ERR_ARG, "wgpt_decode_greedy: token id %d outside [0, %d)", token, m->V);
  if (steps < 1 || !out_tokens) return fail(WGPT_ERR_ARG, "wgpt_decode_greedy: steps >= 1 and out_tokens required");
  if (m->pos + steps > m->ctx)
    return fail(WGPT_ERR_STATE, "wgpt_decode_greedy: %d steps from position %d exceed the context of %d", steps, m->pos, m->ctx);
  const bool persistent = m->decode_mode == 1;
  if (!persistent) {  // (the persistent kernel takes the token as a launch argument)
    m->pin[0] = token;  // every earlier use of the word has completed: each call ends with a synchronisation
    WGPT_HIP(hipMemcpyAsync(m->tok_dev, &m->pin[0], sizeof(int32_t), hipMemcpyHostToDevice, rt().stream));
    int rc = upload_position(m);
    if (rc) return rc;
  }
  WGPT_HIP(hipEventRecord(m->ev0, rt().stream));
  if (persistent) {
    int rc = decode_persistent(m, steps, 1, 1.0, nullptr, token, true);
    if (rc) return rc;
  } else {
    for (int i = 0; i < steps; ++i) {
      int rc = decode_token_blocks(m, m->pos + i);  // advances the device's position itself
      if (rc) return rc;
      LAUNCH(launch_argmax(m->V, m->logits, m->tok_dev, m->out_tok_dev, i, rt().stream));
    }
  }
  {
    int rc = finish_steps(m, out_tokens, m->out_tok_dev, steps, logits);
    if (rc) return rc;
  }
  if (persistent) {
    int rc = check_persistent(m);
    if (rc) return rc;
  }
  m->pos += steps;
  return WGPT_OK;
}

int wgpt_decode_sample(wgpt_model h, int32_t token, int steps, int top_k, double temperature, const double* u,
                       int32_t* out_tokens, float* logits) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  m->res_host_done = m->res_host_logits = false;  // (left set by a call that failed between its launch and its read-back)
  m->x_rows = 0;
  if (!m->finalized) return fail(WGPT_ERR_STATE, "wgpt_decode_sample: model not finalised");
  if (token < 0 || token >= m->V) return fail(WGPT_ERR_ARG, "wgpt_decode_sample: token id %d outside [0, %d)", token, m->V);
  if (steps < 1 || !out_tokens || !u) return fail(WGPT_ERR_ARG, "wgpt_decode_sample: steps >= 1, u and out_tokens required");
  if (top_k < 1 || top_k > SAMPLE_MAX_K) return fail(WGPT_ERR_ARG, "wgpt_decode_sample: top_k must be in [1, %d]", SAMPLE_MAX_K);
  if (m->V > SAMPLE_MAX_V) return fail(WGPT_ERR_ARG, "wgpt_decode_sample: vocabulary above %d", SAMPLE_MAX_V);
  if (!(temperature > 0.0)) return fail(WGPT_ERR_ARG, "wgpt_decode_sample: temperature must be positive");
  for (int i = 0; i < steps; ++i)
    if (!(u[i] >= 0.0 && u[i] < 1.0)) return fail(WGPT_ERR_ARG, "wgpt_decode_sample: u[%d] must be in [0, 1)", i);
  if (m->pos + steps > m->ctx)
    return fail(WGPT_ERR_STATE, "wgpt_decode_sample: %d steps from position %d exceed the context of %d", steps, m->pos, m->ctx);
  WGPT_HIP(hipMemcpyAsync(m->tok_dev, &token, sizeof(int32_t), hipMemcpyHostToDevice, rt().stream));
  WGPT_HIP(hipMemcpyAsync(m->u_dev, u, sizeof(double) * (size_t)steps, hipMemcpyHostToDevice, rt().stream));
  const bool persistent = m->decode_mode == 1;
  if (!persistent) {
    int rc0 = upload_position(m);
    if (rc0) return rc0;
  }
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  WGPT_HIP(hipEventRecord(m->ev0, rt().stream));
  const int k = top_k < m->V ? top_k : m->V;
  // up to PD_TOPK candidates the persistent kernel selects and samples itself, all steps in one launch
  const bool in_kernel = persistent && k <= PD_TOPK;
  // The cache position is committed only when the whole call has succeeded (as wgpt_decode and
  // wgpt_decode_greedy do): after a failure the caller's history is unchanged, so a retry must find the
  // model where the call started. A step of the loop below reads m->pos; it is restored on every error path.
  const int pos_before = m->pos;
  int rc = WGPT_OK;
  if (in_kernel) {
    rc = decode_persistent(m, steps, k, temperature, m->u_dev, token, true);
  } else {
    for (int i = 0; i < steps && rc == WGPT_OK; ++i) {
      // one token per launch: the sampled id in tok_dev[0] is the next launch's input
      rc = persistent ? decode_persistent(m, 1) : decode_token_blocks(m, m->pos);
      if (rc == WGPT_OK) {
        hipError_t e = launch_sample_topk(m->V, k, temperature, m->u_dev + i, m->logits, m->tok_dev, m->out_samp_dev, i, nullptr, nullptr, rt().stream);
        if (e != hipSuccess) rc = fail(WGPT_ERR_HIP, "launch_sample_topk: %s", hipGetErrorString(e));
      }
      m->pos += 1;
    }
  }
  m->pos = pos_before;
  if (rc) {
    (void)hipStreamSynchronize(rt().stream);
    return rc;
  }
  if ((rc = finish_steps(m, out_tokens, in_kernel ? m->out_tok_dev : m->out_samp_dev, steps, logits))) {
    m->pos = pos_before;
    return rc;
  }
  if (persistent && (rc = check_persistent(m))) return rc;
  m->pos = pos_before + steps;
  return WGPT_OK;
}

// One timed launch of `steps` greedy steps from position p0 (token 0), for the delay search: GPU milliseconds, or a
// negative value when the launch failed. The key/value rows it writes are rows that every later call writes before it
// reads them (a model's position is 0 while this runs).
static float timed_trial(Model* m, int p0, int steps) {
  m->pos = p0;
  if (hipEventRecord(m->ev0, rt().stream) != hipSuccess) return -1.f;
  if (decode_persistent(m, steps, 1, 1.0, nullptr, 0, false) != WGPT_OK) return -1.f;
  if (hipEventRecord(m->ev1, rt().stream) != hipSuccess) return -1.f;
  if (hipMemcpyAsync(&m->pin[1], m->perr, sizeof(int), hipMemcpyDeviceToHost, rt().stream) != hipSuccess) return -1.f;
  if (hipStreamSynchronize(rt().stream) != hipSuccess) return -1.f;
  m->pos = 0;
  if (m->pin[1] != 0) return -1.f;
  float ms = -1.f;
  if (hipEventElapsedTime(&ms, m->ev0, m->ev1) != hipSuccess) return -1.f;
  return ms;
}

int wgpt_model_tune_poll_delays(wgpt_model h, int rounds, int32_t* chosen, float* ms_before, float* ms_after) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (!m->finalized) return fail(WGPT_ERR_STATE, "wgpt_model_tune_poll_delays: model not finalised");
  if (!m->persist_ok || m->decode_mode != 1)
    return fail(WGPT_ERR_STATE, "wgpt_model_tune_poll_delays: the persistent decode kernel is not in use for this model");
  if (m->pos != 0) return fail(WGPT_ERR_STATE, "wgpt_model_tune_poll_delays: a context is in use (position %d); call it before the first prefill or after wgpt_model_reset_cache", m->pos);
  if (rounds < 0 || rounds > 8) return fail(WGPT_ERR_ARG, "wgpt_model_tune_poll_delays: rounds must be in [0, 8]");
  m->res_host_done = m->res_host_logits = false;
  m->x_rows = 0;
  // a trial is two launches, at three tenths and at three quarters of the context (the attention exchange's best
  // delays move with the context length: a row found at one length loses at another), together long enough (about
  // 5 ms) that the event clock's granularity does not matter
  const int pa = m->ctx * 3 / 10, pb = m->ctx * 3 / 4;
  int steps = m->ctx - pb < 8 ? m->ctx - pb : 8;
  if (steps < 1 || pa < 1) return fail(WGPT_ERR_STATE, "wgpt_model_tune_poll_delays: context too short");
  const auto timed_pair = [&](int n) {
    const float a = timed_trial(m, pa, n);
    if (a < 0) return -1.f;
    const float b = timed_trial(m, pb, n);
    return b < 0 ? -1.f : a + b;
  };
  const auto failed = [&](const int* restore) -> int {
    for (int i = 0; i < 7; ++i) m->pa.delay[i] = restore[i];
    m->pos = 0;
    if (m->pin[1] != 0) { (void)check_persistent(m); return WGPT_ERR_DEVICE; }
    return fail(WGPT_ERR_DEVICE, "wgpt_model_tune_poll_delays: a trial launch failed");
  };
  int start[7];
  for (int i = 0; i < 7; ++i) start[i] = m->pa.delay[i];
  float t = timed_pair(steps);
  if (t < 0) return failed(start);
  {
    const float per_step = t / (2 * steps);
    int want = per_step > 0 ? (int)(2.5f / per_step) : 32;
    want = want < 8 ? 8 : (want > 32 ? 32 : want);
    steps = m->ctx - pb < want ? m->ctx - pb : want;
    if (pb - pa < steps) steps = pb - pa;
  }
  const auto measure = [&](int reps) {
    float best = 1e30f;
    for (int r = 0; r < reps; ++r) {
      const float v = timed_pair(steps);
      if (v < 0) return -1.f;
      best = v < best ? v : best;
    }
    return best;
  };
  const float before = measure(5);
  if (before < 0) return failed(start);
  // coordinate descent, the delays with the steepest curves first; a move must gain more than the run-to-run noise
  static const int order[7] = {3, 2, 0, 4, 5, 6, 1};
  static const int moves[4] = {-8, -4, 4, 8};
  float cur = before;
  for (int round = 0; round < rounds; ++round) {
    bool moved = false;
    for (int oi = 0; oi < 7; ++oi) {
      const int c = order[oi];
      const int here = m->pa.delay[c];
      cur = measure(3);
      if (cur < 0) return failed(start);
      int best_v = here;
      float best_t = cur * 0.997f;
      for (int mv : moves) {
        const int v = here + mv;
        if (v < 0 || v > 1024) continue;
        m->pa.delay[c] = v;
        const float tv = measure(3);
        if (tv < 0) return failed(start);
        if (tv < best_t) { best_t = tv; best_v = v; }
      }
      m->pa.delay[c] = best_v;
      moved = moved || best_v != here;
    }
    if (!moved) break;
  }
  // the found row against the starting one, alternating: kept only when it wins by more than the noise
  int found[7];
  bool differs = false;
  for (int i = 0; i < 7; ++i) { found[i] = m->pa.delay[i]; differs = differs || found[i] != start[i]; }
  float t_start = before, t_found = before;
  if (differs) {
    t_start = t_found = 1e30f;
    for (int r = 0; r < 4; ++r) {
      for (int i = 0; i < 7; ++i) m->pa.delay[i] = start[i];
      float v = measure(2);
      if (v < 0) return failed(start);
      t_start = v < t_start ? v : t_start;
      for (int i = 0; i < 7; ++i) m->pa.delay[i] = found[i];
      v = measure(2);
      if (v < 0) return failed(start);
      t_found = v < t_found ? v : t_found;
    }
    if (!(t_found < t_start * 0.995f)) {
      for (int i = 0; i < 7; ++i) m->pa.delay[i] = start[i];
      t_found = t_start;
    }
  }
  m->pos = 0;
  if (chosen) for (int i = 0; i < 7; ++i) chosen[i] = m->pa.delay[i];
  if (ms_before) *ms_before = t_start / (2 * steps);
  if (ms_after) *ms_after = t_found / (2 * steps);
  return WGPT_OK;
}

int wgpt_model_poll_delays(wgpt_model h, int32_t* out) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m || !out) return fail(WGPT_ERR_ARG, "wgpt_model_poll_delays: NULL argument");
  if (!m->finalized || !m->persist_ok) return fail(WGPT_ERR_STATE, "wgpt_model_poll_delays: the persistent decode kernel is not set up for this model");
  for (int i = 0; i < 7; ++i) out[i] = m->pa.delay[i];
  return WGPT_OK;
}

int wgpt_model_reset_cache(wgpt_model h) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  m->pos = 0;
  m->tap_T = 0;
  m->x_rows = 0;
  return WGPT_OK;
}

int wgpt_model_position(wgpt_model h, int* pos) {
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (pos) *pos = m->pos;
  return WGPT_OK;
}

int wgpt_model_tap(wgpt_model h, const char* name, float* out, size_t n_floats) {
  WGPT_REQUIRE_INIT();
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (!name || !out) return fail(WGPT_ERR_ARG, "wgpt_model_tap: NULL argument");
  if (!m->finalized) return fail(WGPT_ERR_STATE, "wgpt_model_tap: model not finalised");
  const std::string n = name;
  const size_t d = m->d;
  const float* src = nullptr;
  size_t count = 0;
  int layer = -1;
  char which[16] = "";
  if (sscanf(name, "kv%d_%15s", &layer, which) == 2 && layer >= 0 && layer < m->L && (!strcmp(which, "k") || !strcmp(which, "v"))) {
    // the cache is head-major [H][ctx][hs]: gather rows 0..pos-1 into [pos, d]
    count = (size_t)m->pos * d;
    if (n_floats != count) return fail(WGPT_ERR_ARG, "wgpt_model_tap: '%s' holds %zu floats, caller asked for %zu", name, count, n_floats);
    if (count == 0) return WGPT_OK;
    const float* base = m->kv + ((size_t)layer * 2 + (which[0] == 'v' ? 1 : 0)) * m->ctx * d;
    for (int h2 = 0; h2 < m->H; ++h2)
      WGPT_HIP(hipMemcpy2DAsync(out + (size_t)h2 * m->hs, sizeof(float) * d, base + (size_t)h2 * m->ctx * m->hs,
                                sizeof(float) * m->hs, sizeof(float) * m->hs, (size_t)m->pos, hipMemcpyDeviceToHost, rt().stream));
    WGPT_HIP(hipStreamSynchronize(rt().stream));
    return WGPT_OK;
  } else if (n == "residual") {
    // the residual stream after the last layer as the last prefill left it: what the reference copies into
    // GPT.externalBuffer (model.js:211-222); needs no WGPT_FLAG_TAPS
    if (m->x_rows == 0) return fail(WGPT_ERR_STATE, "wgpt_model_tap: 'residual' holds the rows of the last wgpt_prefill until the next decode step");
    src = m->x;
    count = (size_t)m->x_rows * d;
  } else {
    if (!m->taps || m->tap_T == 0) return fail(WGPT_ERR_STATE, "wgpt_model_tap: no taps recorded (WGPT_FLAG_TAPS and a prefill are needed)");
    const size_t T = m->tap_T;
    long index = -1;
    if (n == "tok_pos_emb") index = 0;
    else if (n == "ln_f") index = 1 + 6 * (long)m->L;
    else if (sscanf(name, "block%d_%15s", &layer, which) == 2 && layer >= 0 && layer < m->L) {
      const char* subs[6] = {"ln1", "attn", "r1", "ln2", "mlp", "r2"};
      for (int k = 0; k < 6; ++k)
        if (!strcmp(which, subs[k])) index = 1 + 6 * (long)layer + k;
    }
    if (index < 0) return fail(WGPT_ERR_ARG, "wgpt_model_tap: unknown tap '%s'", name);
    src = m->taps + (size_t)index * T * d;
    count = T * d;
  }
  if (n_floats != count) return fail(WGPT_ERR_ARG, "wgpt_model_tap: '%s' holds %zu floats, caller asked for %zu", name, count, n_floats);
  if (count == 0) return WGPT_OK;
  WGPT_HIP(hipMemcpyAsync(out, src, sizeof(float) * count, hipMemcpyDeviceToHost, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  return WGPT_OK;
}

int wgpt_model_last_gpu_ms(wgpt_model h, float* ms) {
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (ms) *ms = m->last_ms;
  return WGPT_OK;
}

int wgpt_model_decode_bytes(wgpt_model h, int t, uint64_t* bytes) {
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (t < 0 || t > m->ctx) return fail(WGPT_ERR_ARG, "wgpt_model_decode_bytes: t outside [0, n_ctx]");
  const uint64_t d = m->d, L = m->L, V = m->V;
  uint64_t w;
  if (m->p.weight_dtype == 0) w = 4 * (L * (12 * d * d + 13 * d) + V * d + 2 * d);
  else w = L * (12 * d * d) + 4 * (L * (13 * d + 9 * d) + V * d + 2 * d);
  if (bytes) *bytes = w + 8 * L * d * (uint64_t)t;
  return WGPT_OK;
}

int wgpt_model_set_decode_mode(wgpt_model h, int mode) {
  Model* m = find_model(h);
  if (!m) return WGPT_ERR_ARG;
  if (mode != 0 && mode != 1) return fail(WGPT_ERR_ARG, "wgpt_model_set_decode_mode: unknown mode %d", mode);
  if (mode == 1 && !m->persist_ok)
    return fail(WGPT_ERR_STATE, "wgpt_model_set_decode_mode: the persistent decode path is not available for this model "
                                "(needs head size 64, a supported width and 256 compute units)");
  m->decode_mode = mode;
  return WGPT_OK;
}

int wgpt_model_destroy(wgpt_model h) {
  WGPT_REQUIRE_INIT();
  auto it = models().find(h);
  if (it == models().end()) return fail(WGPT_ERR_ARG, "wgpt_model_destroy: unknown model handle %llu", (unsigned long long)h);
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  destroy_model(it->second);
  models().erase(it);
  return WGPT_OK;
}

}  // extern "C"
