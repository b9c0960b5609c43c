// Device-side state of one loaded model.
#ifndef WGPT_MODEL_H
#define WGPT_MODEL_H

#include <hip/hip_runtime.h>

#include <cstdint>
#include <vector>

#include "../../include/webgpt_amd.h"
#include "decode_persistent.h"

namespace wgpt {

// One linear layer's weight: fp32 [K,N], or int8 words [K,N/4] + per-column scale [N].
struct LinW {
  float* w = nullptr;
  int32_t* q = nullptr;
  float* s = nullptr;
};

struct LayerW {
  float *ln1_g = nullptr, *ln1_b = nullptr, *ln2_g = nullptr, *ln2_b = nullptr;
  LinW attn, proj, fc, fc2;  // c_attn [d,3d], c_proj [d,d], c_fc [d,4d], mlp c_proj [4d,d]
  float *attn_b = nullptr, *proj_b = nullptr, *fc_b = nullptr, *fc2_b = nullptr;
};

struct Model {
  wgpt_params p{};
  int L = 0, H = 0, d = 0, hs = 0, ctx = 0, V = 0, maxT = 0;
  bool finalized = false;
  int decode_mode = 0;
  int pos = 0;     // positions held by the KV cache
  int tap_T = 0;   // rows of the recorded taps (0 = none)
  int x_rows = 0;  // rows of the residual stream the last prefill left in x (0 once a decode step has run)

  float *wte = nullptr, *wpe = nullptr, *lnf_g = nullptr, *lnf_b = nullptr;
  std::vector<LayerW> layers;

  float* kv = nullptr;  // [L][2][H][ctx][hs]: keys then values of each layer, head-major
  // activations for up to maxT rows
  float *x = nullptr, *ln = nullptr, *qkv = nullptr, *att = nullptr, *tmp = nullptr, *h = nullptr;
  float* logits = nullptr;       // [V]
  float* part = nullptr;         // GEMV partial sums
  float* dq = nullptr;           // fp32 scratch for a dequantised int8 matrix (prefill)
  float* taps = nullptr;         // [(2+6L)][maxT][d]
  int32_t* tok_dev = nullptr;    // [maxT] token ids of the current call
  int32_t* out_tok_dev = nullptr;  // [ctx] ids chosen by the greedy loop
  int32_t* out_samp_dev = nullptr; // [ctx] ids chosen by the sampling loop
  double* u_dev = nullptr;         // [ctx] uniform draws of the sampling loop

  // persistent whole-token decode (decode_mode 1): slab-layout weights, exchange buffers
  bool slabs_ok = false;   // pa.slabs / pa.lparams are built (every shape)
  bool persist_ok = false;
  PersistentArgs pa{};
  int* perr = nullptr;       // device error word of the persistent kernel
  // pinned host words (hipHostMalloc): [0] the token of a single-step call on its way to the device,
  // [1] the error word on its way back, so that a decode call needs one stream synchronisation, [2] the cache position
  // on its way to pos_dev
  int32_t* pin = nullptr;
  float* logits_pin = nullptr;  // pinned host copy of the logits of the last call (V floats and the error word behind them)
  int32_t* ids_pin = nullptr;   // pinned host copy of the ids of a multi-step call (ctx ints)
  // set by a persistent launch that writes its results to pinned memory itself, cleared by the read-back behind it:
  // pin[1] holds the error word (or still -1: the kernel did not reach its end); logits_pin holds the logits
  bool res_host_done = false, res_host_logits = false;
  unsigned epoch = 0;        // last epoch published by earlier launches

  // decode with one launch per block (decode_mode 0): the token's launches read the cache position from pos_dev and
  // are recorded once as a HIP graph that every later token replays
  int* pos_dev = nullptr;
  hipGraph_t token_graph = nullptr;
  hipGraphExec_t token_graph_exec = nullptr;
  bool token_graph_tried = false;
  // attention of a decode token over a cache of more than one slice: (output, maximum, sum) per head and slice
  float* att_part = nullptr;
  int att_nslice = 1;

  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  float last_ms = 0.f;
  std::vector<void*> allocs;
};

void destroy_all_models();

}  // namespace wgpt

#endif
