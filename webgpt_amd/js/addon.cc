// Node N-API addon: the JavaScript host's door to the C ABI of include/webgpt_amd.h.
//
// The addon does not link HIP. It dlopen()s libwebgpt_amd.so (next to the package)
// and forwards calls; every non-zero return of the library becomes a thrown Error
// carrying wgpt_last_error(), which is how the reference reports precondition
// failures (throw new Error(...), instructions.js:79,158).
//
// Build: g++ -O2 -std=c++17 -shared -fPIC -I/usr/include/node addon.cc -o wgpt_addon.node -ldl
#include <dlfcn.h>
#include <node_api.h>

#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/webgpt_amd.h"

namespace {

void* g_lib = nullptr;

#define WGPT_FUNCS(X)                                                                                   \
  X(wgpt_init) X(wgpt_shutdown) X(wgpt_last_error) X(wgpt_device_info) X(wgpt_alloc) X(wgpt_free)       \
  X(wgpt_buf_size) X(wgpt_upload) X(wgpt_download) X(wgpt_copy) X(wgpt_sync) X(wgpt_matmul_bias)        \
  X(wgpt_matmul_bias_i8) X(wgpt_dequant_i8) X(wgpt_residual) X(wgpt_layernorm) X(wgpt_softmax)          \
  X(wgpt_gelu) X(wgpt_embed) X(wgpt_deembed) X(wgpt_attention) X(wgpt_model_create)                     \
  X(wgpt_model_set_tensor) X(wgpt_model_finalize) X(wgpt_prefill) X(wgpt_decode) X(wgpt_decode_greedy)  \
  X(wgpt_model_reset_cache) X(wgpt_model_position) X(wgpt_model_tap) X(wgpt_model_last_gpu_ms)          \
  X(wgpt_model_decode_bytes) X(wgpt_model_set_decode_mode) X(wgpt_model_destroy) X(wgpt_synth_normal)   \
  X(wgpt_synth_tokens) X(wgpt_synth_int8_packed) X(wgpt_synth_uniform) X(wgpt_synth_tensor_id)   \
  X(wgpt_decode_sample) X(wgpt_sample_topk) X(wgpt_matmul_bias_noalloc) X(wgpt_softmax_t) X(wgpt_transpose)   \
  X(wgpt_model_tune_poll_delays) X(wgpt_model_poll_delays)

#define DECL(name) decltype(&::name) p_##name = nullptr;
WGPT_FUNCS(DECL)
#undef DECL

napi_value throw_error(napi_env env, const char* msg) {
  napi_throw_error(env, nullptr, msg);
  return nullptr;
}

// Throws the library's last error when rc != 0. Returns true when an exception is pending.
bool failed(napi_env env, int rc) {
  if (rc == 0) return false;
  const char* msg = p_wgpt_last_error ? p_wgpt_last_error() : "webgpt_amd: call failed";
  napi_throw_error(env, nullptr, msg && *msg ? msg : "webgpt_amd: call failed");
  return true;
}

struct Args {
  napi_env env;
  size_t argc = 24;
  napi_value argv[24];
  bool ok = true;
  Args(napi_env e, napi_callback_info info) : env(e) {
    if (napi_get_cb_info(env, info, &argc, argv, nullptr, nullptr) != napi_ok) ok = false;
  }
  double num(size_t i) {
    double v = 0;
    if (i >= argc || napi_get_value_double(env, argv[i], &v) != napi_ok) {
      ok = false;
      napi_throw_type_error(env, nullptr, "webgpt_amd: numeric argument expected");
    }
    return v;
  }
  int i32(size_t i) { return (int)num(i); }
  uint64_t u64(size_t i) { return (uint64_t)num(i); }
  std::string str(size_t i) {
    char buf[512];
    size_t n = 0;
    if (i >= argc || napi_get_value_string_utf8(env, argv[i], buf, sizeof(buf), &n) != napi_ok) {
      ok = false;
      napi_throw_type_error(env, nullptr, "webgpt_amd: string argument expected");
      return "";
    }
    return std::string(buf, n);
  }
  // Bytes of a TypedArray / ArrayBuffer / Buffer argument.
  bool bytes(size_t i, void** data, size_t* len) {
    if (i >= argc) { ok = false; return false; }
    bool is = false;
    napi_is_typedarray(env, argv[i], &is);
    if (is) {
      napi_typedarray_type type;
      size_t count, off;
      napi_value ab;
      if (napi_get_typedarray_info(env, argv[i], &type, &count, data, &ab, &off) != napi_ok) { ok = false; return false; }
      static const size_t width[] = {1, 1, 1, 2, 2, 4, 4, 4, 8, 8, 8};
      *len = count * width[type];
      return true;
    }
    napi_is_arraybuffer(env, argv[i], &is);
    if (is) return napi_get_arraybuffer_info(env, argv[i], data, len) == napi_ok;
    napi_is_buffer(env, argv[i], &is);
    if (is) return napi_get_buffer_info(env, argv[i], data, len) == napi_ok;
    ok = false;
    napi_throw_type_error(env, nullptr, "webgpt_amd: TypedArray, ArrayBuffer or Buffer expected");
    return false;
  }
};

napi_value undefined(napi_env env) {
  napi_value v;
  napi_get_undefined(env, &v);
  return v;
}
napi_value number(napi_env env, double d) {
  napi_value v;
  napi_create_double(env, d, &v);
  return v;
}

#define FN(name) napi_value name(napi_env env, napi_callback_info info)

FN(Init) { Args a(env, info); int dev = a.i32(0); if (!a.ok) return nullptr; if (failed(env, p_wgpt_init(dev))) return nullptr; return undefined(env); }
FN(Shutdown) { if (failed(env, p_wgpt_shutdown())) return nullptr; return undefined(env); }
FN(Sync) { if (failed(env, p_wgpt_sync())) return nullptr; return undefined(env); }

FN(DeviceInfo) {
  char name[128] = "";
  int cus = 0;
  uint64_t hbm = 0;
  if (failed(env, p_wgpt_device_info(name, sizeof(name), &cus, &hbm))) return nullptr;
  napi_value o, s;
  napi_create_object(env, &o);
  napi_create_string_utf8(env, name, NAPI_AUTO_LENGTH, &s);
  napi_set_named_property(env, o, "name", s);
  napi_set_named_property(env, o, "computeUnits", number(env, cus));
  napi_set_named_property(env, o, "hbmBytes", number(env, (double)hbm));
  return o;
}

FN(Alloc) {
  Args a(env, info);
  const double bytes = a.num(0);
  if (!a.ok) return nullptr;
  wgpt_buf h = 0;
  if (failed(env, p_wgpt_alloc((size_t)bytes, &h))) return nullptr;
  return number(env, (double)h);
}
FN(Free) { Args a(env, info); uint64_t h = a.u64(0); if (!a.ok) return nullptr; if (failed(env, p_wgpt_free(h))) return nullptr; return undefined(env); }

FN(Upload) {  // (handle, offsetBytes, data)
  Args a(env, info);
  uint64_t h = a.u64(0);
  size_t off = (size_t)a.num(1);
  void* data;
  size_t len;
  if (!a.ok || !a.bytes(2, &data, &len)) return nullptr;
  if (failed(env, p_wgpt_upload(h, off, data, len))) return nullptr;
  return undefined(env);
}
FN(Download) {  // (handle, offsetBytes, bytes) -> ArrayBuffer
  Args a(env, info);
  uint64_t h = a.u64(0);
  size_t off = (size_t)a.num(1), len = (size_t)a.num(2);
  if (!a.ok) return nullptr;
  void* data;
  napi_value ab;
  if (napi_create_arraybuffer(env, len, &data, &ab) != napi_ok) return throw_error(env, "webgpt_amd: out of memory");
  if (failed(env, p_wgpt_download(data, h, off, len))) return nullptr;
  return ab;
}
FN(Copy) {  // (dst, dstOff, src, srcOff, bytes)
  Args a(env, info);
  uint64_t d = a.u64(0), s = a.u64(2);
  size_t doff = (size_t)a.num(1), soff = (size_t)a.num(3), n = (size_t)a.num(4);
  if (!a.ok) return nullptr;
  if (failed(env, p_wgpt_copy(d, doff, s, soff, n))) return nullptr;
  return undefined(env);
}

FN(MatmulBias) { Args a(env, info); int M = a.i32(0), N = a.i32(1), K = a.i32(2); uint64_t A = a.u64(3), W = a.u64(4), b = a.u64(5), C = a.u64(6); if (!a.ok) return nullptr; if (failed(env, p_wgpt_matmul_bias(M, N, K, A, W, b, C))) return nullptr; return undefined(env); }
FN(MatmulBiasNoAlloc) { Args a(env, info); int M = a.i32(0), N = a.i32(1), K = a.i32(2); uint64_t A = a.u64(3), W = a.u64(4), b = a.u64(5), C = a.u64(6); if (!a.ok) return nullptr; if (failed(env, p_wgpt_matmul_bias_noalloc(M, N, K, A, W, b, C))) return nullptr; return undefined(env); }
FN(MatmulBiasI8) { Args a(env, info); int M = a.i32(0), N = a.i32(1), K = a.i32(2); uint64_t A = a.u64(3), W = a.u64(4), s = a.u64(5), b = a.u64(6), C = a.u64(7); if (!a.ok) return nullptr; if (failed(env, p_wgpt_matmul_bias_i8(M, N, K, A, W, s, b, C))) return nullptr; return undefined(env); }
FN(DequantI8) { Args a(env, info); int K = a.i32(0), N = a.i32(1); uint64_t q = a.u64(2), s = a.u64(3), w = a.u64(4); if (!a.ok) return nullptr; if (failed(env, p_wgpt_dequant_i8(K, N, q, s, w))) return nullptr; return undefined(env); }
FN(Residual) { Args a(env, info); int M = a.i32(0), N = a.i32(1); uint64_t x = a.u64(2), y = a.u64(3), o = a.u64(4); if (!a.ok) return nullptr; if (failed(env, p_wgpt_residual(M, N, x, y, o))) return nullptr; return undefined(env); }
FN(LayerNorm) { Args a(env, info); int M = a.i32(0), N = a.i32(1); uint64_t x = a.u64(2), g = a.u64(3), b = a.u64(4), o = a.u64(5); if (!a.ok) return nullptr; if (failed(env, p_wgpt_layernorm(M, N, x, g, b, o))) return nullptr; return undefined(env); }
FN(Softmax) { Args a(env, info); int M = a.i32(0), N = a.i32(1); uint64_t x = a.u64(2), o = a.u64(3); if (!a.ok) return nullptr; if (failed(env, p_wgpt_softmax(M, N, x, o))) return nullptr; return undefined(env); }
FN(SoftmaxT) { Args a(env, info); int M = a.i32(0), N = a.i32(1); uint64_t x = a.u64(2), o = a.u64(3); if (!a.ok) return nullptr; if (failed(env, p_wgpt_softmax_t(M, N, x, o))) return nullptr; return undefined(env); }
FN(Transpose) { Args a(env, info); int M = a.i32(0), N = a.i32(1); uint64_t x = a.u64(2), o = a.u64(3); if (!a.ok) return nullptr; if (failed(env, p_wgpt_transpose(M, N, x, o))) return nullptr; return undefined(env); }
FN(Gelu) { Args a(env, info); int M = a.i32(0), N = a.i32(1); uint64_t x = a.u64(2), o = a.u64(3); if (!a.ok) return nullptr; if (failed(env, p_wgpt_gelu(M, N, x, o))) return nullptr; return undefined(env); }
FN(Embed) {  // (Int32Array idx, T, d, V, wte, wpe, out)
  Args a(env, info);
  void* data;
  size_t len;
  if (!a.bytes(0, &data, &len)) return nullptr;
  int T = a.i32(1), d = a.i32(2), V = a.i32(3);
  uint64_t wte = a.u64(4), wpe = a.u64(5), out = a.u64(6);
  if (!a.ok) return nullptr;
  if (len < sizeof(int32_t) * (size_t)(T > 0 ? T : 0)) return throw_error(env, "wgpt_embed: idx holds fewer than T ids");
  if (failed(env, p_wgpt_embed((const int32_t*)data, T, d, V, wte, wpe, out))) return nullptr;
  return undefined(env);
}
FN(DeEmbed) { Args a(env, info); int d = a.i32(0), V = a.i32(1), T = a.i32(2); uint64_t x = a.u64(3), w = a.u64(4), o = a.u64(5); if (!a.ok) return nullptr; if (failed(env, p_wgpt_deembed(d, V, T, x, w, o))) return nullptr; return undefined(env); }
FN(Attention) {
  Args a(env, info);
  int T = a.i32(0), d = a.i32(1);
  float scale = (float)a.num(2);
  int H = a.i32(3), hs = a.i32(4);
  uint64_t b[10];
  for (int i = 0; i < 10; ++i) b[i] = a.u64(5 + i);
  if (!a.ok) return nullptr;
  if (failed(env, p_wgpt_attention(T, d, scale, H, hs, b[0], b[1], b[2], b[3], b[4], b[5], b[6], b[7], b[8], b[9]))) return nullptr;
  return undefined(env);
}

FN(ModelCreate) {  // (n_layer, n_head, n_embd, n_ctx, vocab_size, weight_dtype, max_prefill, flags) -> handle
  Args a(env, info);
  wgpt_params p;
  p.n_layer = a.i32(0); p.n_head = a.i32(1); p.n_embd = a.i32(2); p.n_ctx = a.i32(3); p.vocab_size = a.i32(4);
  p.weight_dtype = a.i32(5); p.max_prefill = a.i32(6); p.flags = a.i32(7);
  if (!a.ok) return nullptr;
  wgpt_model m = 0;
  if (failed(env, p_wgpt_model_create(&p, &m))) return nullptr;
  return number(env, (double)m);
}
FN(ModelSetTensor) {  // (model, name, data)
  Args a(env, info);
  uint64_t m = a.u64(0);
  std::string name = a.str(1);
  void* data;
  size_t len;
  if (!a.ok || !a.bytes(2, &data, &len)) return nullptr;
  if (failed(env, p_wgpt_model_set_tensor(m, name.c_str(), data, len))) return nullptr;
  return undefined(env);
}
FN(ModelFinalize) { Args a(env, info); uint64_t m = a.u64(0); if (!a.ok) return nullptr; if (failed(env, p_wgpt_model_finalize(m))) return nullptr; return undefined(env); }
FN(ModelDestroy) { Args a(env, info); uint64_t m = a.u64(0); if (!a.ok) return nullptr; if (failed(env, p_wgpt_model_destroy(m))) return nullptr; return undefined(env); }
FN(ModelResetCache) { Args a(env, info); uint64_t m = a.u64(0); if (!a.ok) return nullptr; if (failed(env, p_wgpt_model_reset_cache(m))) return nullptr; return undefined(env); }
FN(ModelSetDecodeMode) { Args a(env, info); uint64_t m = a.u64(0); int mode = a.i32(1); if (!a.ok) return nullptr; if (failed(env, p_wgpt_model_set_decode_mode(m, mode))) return nullptr; return undefined(env); }
FN(ModelPosition) { Args a(env, info); uint64_t m = a.u64(0); if (!a.ok) return nullptr; int pos = 0; if (failed(env, p_wgpt_model_position(m, &pos))) return nullptr; return number(env, pos); }
FN(ModelLastGpuMs) { Args a(env, info); uint64_t m = a.u64(0); if (!a.ok) return nullptr; float ms = 0; if (failed(env, p_wgpt_model_last_gpu_ms(m, &ms))) return nullptr; return number(env, ms); }
FN(ModelDecodeBytes) { Args a(env, info); uint64_t m = a.u64(0); int t = a.i32(1); if (!a.ok) return nullptr; uint64_t b = 0; if (failed(env, p_wgpt_model_decode_bytes(m, t, &b))) return nullptr; return number(env, (double)b); }

// seven poll delays (and, after a search, the milliseconds per token before and after it) as a Float32Array
FN(ModelPollDelays) {  // (model) -> Float32Array[7]
  Args a(env, info);
  uint64_t m = a.u64(0);
  if (!a.ok) return nullptr;
  int32_t row[7];
  if (failed(env, p_wgpt_model_poll_delays(m, row))) return nullptr;
  napi_value ab, ta;
  void* p;
  if (napi_create_arraybuffer(env, 7 * sizeof(float), &p, &ab) != napi_ok) return nullptr;
  napi_create_typedarray(env, napi_float32_array, 7, ab, 0, &ta);
  for (int i = 0; i < 7; ++i) ((float*)p)[i] = (float)row[i];
  return ta;
}
FN(ModelTunePollDelays) {  // (model, rounds) -> Float32Array[9]: the row kept, ms/token before, ms/token after
  Args a(env, info);
  uint64_t m = a.u64(0);
  int rounds = a.i32(1);
  if (!a.ok) return nullptr;
  int32_t row[7];
  float before = 0, after = 0;
  if (failed(env, p_wgpt_model_tune_poll_delays(m, rounds, row, &before, &after))) return nullptr;
  napi_value ab, ta;
  void* p;
  if (napi_create_arraybuffer(env, 9 * sizeof(float), &p, &ab) != napi_ok) return nullptr;
  napi_create_typedarray(env, napi_float32_array, 9, ab, 0, &ta);
  for (int i = 0; i < 7; ++i) ((float*)p)[i] = (float)row[i];
  ((float*)p)[7] = before;
  ((float*)p)[8] = after;
  return ta;
}

napi_value new_f32(napi_env env, size_t count, float** data) {
  napi_value ab, ta;
  void* p;
  if (napi_create_arraybuffer(env, count * sizeof(float), &p, &ab) != napi_ok) return nullptr;
  napi_create_typedarray(env, napi_float32_array, count, ab, 0, &ta);
  *data = (float*)p;
  return ta;
}

FN(Prefill) {  // (model, Int32Array tokens, vocab) -> Float32Array logits
  Args a(env, info);
  uint64_t m = a.u64(0);
  void* data;
  size_t len;
  if (!a.ok || !a.bytes(1, &data, &len)) return nullptr;
  int V = a.i32(2);
  if (!a.ok) return nullptr;
  float* out;
  napi_value ta = new_f32(env, (size_t)V, &out);
  if (!ta) return throw_error(env, "webgpt_amd: out of memory");
  if (failed(env, p_wgpt_prefill(m, (const int32_t*)data, (int)(len / sizeof(int32_t)), out))) return nullptr;
  return ta;
}
FN(Decode) {  // (model, token, vocab) -> Float32Array logits
  Args a(env, info);
  uint64_t m = a.u64(0);
  int tok = a.i32(1), V = a.i32(2);
  if (!a.ok) return nullptr;
  float* out;
  napi_value ta = new_f32(env, (size_t)V, &out);
  if (!ta) return throw_error(env, "webgpt_amd: out of memory");
  if (failed(env, p_wgpt_decode(m, tok, out))) return nullptr;
  return ta;
}
FN(DecodeGreedy) {  // (model, token, steps) -> Int32Array ids
  Args a(env, info);
  uint64_t m = a.u64(0);
  int tok = a.i32(1), steps = a.i32(2);
  if (!a.ok) return nullptr;
  if (steps < 1) return throw_error(env, "wgpt_decode_greedy: steps >= 1 required");
  napi_value ab, ta;
  void* p;
  if (napi_create_arraybuffer(env, sizeof(int32_t) * (size_t)steps, &p, &ab) != napi_ok) return throw_error(env, "webgpt_amd: out of memory");
  napi_create_typedarray(env, napi_int32_array, (size_t)steps, ab, 0, &ta);
  if (failed(env, p_wgpt_decode_greedy(m, tok, steps, (int32_t*)p, nullptr))) return nullptr;
  return ta;
}
FN(DecodeSample) {  // (model, token, topK, temperature, Float64Array u) -> Int32Array ids, one per draw
  Args a(env, info);
  uint64_t m = a.u64(0);
  int tok = a.i32(1), top_k = a.i32(2);
  double temperature = a.num(3);
  if (!a.ok) return nullptr;
  napi_typedarray_type type;
  size_t steps = 0;
  void* udata = nullptr;
  if (a.argc < 5 || napi_get_typedarray_info(env, a.argv[4], &type, &steps, &udata, nullptr, nullptr) != napi_ok || type != napi_float64_array || steps < 1)
    return throw_error(env, "wgpt_decode_sample: u must be a non-empty Float64Array");
  napi_value ab, ta;
  void* p;
  if (napi_create_arraybuffer(env, sizeof(int32_t) * steps, &p, &ab) != napi_ok) return throw_error(env, "webgpt_amd: out of memory");
  napi_create_typedarray(env, napi_int32_array, steps, ab, 0, &ta);
  if (failed(env, p_wgpt_decode_sample(m, tok, (int)steps, top_k, temperature, (const double*)udata, (int32_t*)p, nullptr))) return nullptr;
  return ta;
}
FN(SampleTopK) {  // (V, topK, temperature, u, logitsBuffer) -> {id, topKIndices: Int32Array, probs: Float64Array}
  Args a(env, info);
  int V = a.i32(0), top_k = a.i32(1);
  double temperature = a.num(2), u = a.num(3);
  uint64_t buf = a.u64(4);
  if (!a.ok) return nullptr;
  if (top_k < 1 || V < 1) return throw_error(env, "wgpt_sample_topk: V and top_k must be positive");
  const size_t k = (size_t)(top_k < V ? top_k : V);
  napi_value ab_i, ta_i, ab_p, ta_p, obj, idv;
  void *pi, *pp;
  if (napi_create_arraybuffer(env, sizeof(int32_t) * k, &pi, &ab_i) != napi_ok || napi_create_arraybuffer(env, sizeof(double) * k, &pp, &ab_p) != napi_ok)
    return throw_error(env, "webgpt_amd: out of memory");
  napi_create_typedarray(env, napi_int32_array, k, ab_i, 0, &ta_i);
  napi_create_typedarray(env, napi_float64_array, k, ab_p, 0, &ta_p);
  int32_t id = 0;
  if (failed(env, p_wgpt_sample_topk(V, top_k, temperature, u, buf, &id, (int32_t*)pi, (double*)pp))) return nullptr;
  napi_create_object(env, &obj);
  napi_create_int32(env, id, &idv);
  napi_set_named_property(env, obj, "id", idv);
  napi_set_named_property(env, obj, "topKIndices", ta_i);
  napi_set_named_property(env, obj, "probs", ta_p);
  return obj;
}
FN(ModelTap) {  // (model, name, nFloats) -> Float32Array
  Args a(env, info);
  uint64_t m = a.u64(0);
  std::string name = a.str(1);
  size_t n = (size_t)a.num(2);
  if (!a.ok) return nullptr;
  float* out;
  napi_value ta = new_f32(env, n, &out);
  if (!ta) return throw_error(env, "webgpt_amd: out of memory");
  if (failed(env, p_wgpt_model_tap(m, name.c_str(), out, n))) return nullptr;
  return ta;
}

FN(SynthNormal) {  // (seed, name, count, std) -> Float32Array
  Args a(env, info);
  uint32_t seed = (uint32_t)a.num(0);
  std::string name = a.str(1);
  size_t n = (size_t)a.num(2);
  double sd = a.num(3);
  if (!a.ok) return nullptr;
  float* out;
  napi_value ta = new_f32(env, n, &out);
  if (!ta) return throw_error(env, "webgpt_amd: out of memory");
  p_wgpt_synth_normal(seed, p_wgpt_synth_tensor_id(name.c_str()), n, sd, out);
  return ta;
}

bool load_library(napi_env env, const char* path) {
  g_lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!g_lib) {
    std::string msg = std::string("webgpt_amd: cannot load ") + path + ": " + dlerror() +
                      " (build it with `make -C webgpt_amd/csrc`; there is no fallback implementation)";
    napi_throw_error(env, nullptr, msg.c_str());
    return false;
  }
#define LOAD(name)                                                               \
  p_##name = reinterpret_cast<decltype(p_##name)>(dlsym(g_lib, #name));          \
  if (!p_##name) {                                                               \
    napi_throw_error(env, nullptr, "webgpt_amd: symbol " #name " missing from the shared library"); \
    return false;                                                                \
  }
  WGPT_FUNCS(LOAD)
#undef LOAD
  return true;
}

FN(Load) {  // (path to libwebgpt_amd.so)
  Args a(env, info);
  std::string path = a.str(0);
  if (!a.ok) return nullptr;
  if (g_lib) return undefined(env);
  if (!load_library(env, path.c_str())) return nullptr;
  return undefined(env);
}

FN(Exports) {  // names of the C-ABI symbols bound by the addon
  napi_value arr;
  napi_create_array(env, &arr);
  uint32_t i = 0;
#define PUSH(name) { napi_value s; napi_create_string_utf8(env, #name, NAPI_AUTO_LENGTH, &s); napi_set_element(env, arr, i++, s); }
  WGPT_FUNCS(PUSH)
#undef PUSH
  return arr;
}

napi_value InitModule(napi_env env, napi_value exports) {
  const struct { const char* name; napi_callback fn; } table[] = {
      {"load", Load}, {"exports", Exports}, {"init", Init}, {"shutdown", Shutdown}, {"sync", Sync}, {"deviceInfo", DeviceInfo},
      {"alloc", Alloc}, {"free", Free}, {"upload", Upload}, {"download", Download}, {"copy", Copy},
      {"wgpt_matmul_bias", MatmulBias}, {"wgpt_matmul_bias_noalloc", MatmulBiasNoAlloc}, {"wgpt_matmul_bias_i8", MatmulBiasI8}, {"wgpt_dequant_i8", DequantI8},
      {"wgpt_residual", Residual}, {"wgpt_layernorm", LayerNorm}, {"wgpt_softmax", Softmax}, {"wgpt_softmax_t", SoftmaxT}, {"wgpt_transpose", Transpose}, {"wgpt_gelu", Gelu},
      {"wgpt_embed", Embed}, {"wgpt_deembed", DeEmbed}, {"wgpt_attention", Attention},
      {"modelCreate", ModelCreate}, {"modelSetTensor", ModelSetTensor}, {"modelFinalize", ModelFinalize},
      {"modelDestroy", ModelDestroy}, {"modelResetCache", ModelResetCache}, {"modelSetDecodeMode", ModelSetDecodeMode},
      {"modelPosition", ModelPosition}, {"modelLastGpuMs", ModelLastGpuMs}, {"modelDecodeBytes", ModelDecodeBytes},
      {"modelPollDelays", ModelPollDelays}, {"modelTunePollDelays", ModelTunePollDelays},
      {"prefill", Prefill}, {"decode", Decode}, {"decodeGreedy", DecodeGreedy}, {"decodeSample", DecodeSample}, {"sampleTopK", SampleTopK}, {"modelTap", ModelTap},
      {"synthNormal", SynthNormal}};
  for (const auto& e : table) {
    napi_value fn;
    napi_create_function(env, e.name, NAPI_AUTO_LENGTH, e.fn, nullptr, &fn);
    napi_set_named_property(env, exports, e.name, fn);
  }
  return exports;
}

}  // namespace

NAPI_MODULE(NODE_GYP_MODULE_NAME, InitModule)
