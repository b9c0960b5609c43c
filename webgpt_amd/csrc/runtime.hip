// Lifecycle, error reporting, device buffers and the synthetic-tensor generator.
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "common.h"
#include "model.h"
#include "wgpt_synth.h"

namespace wgpt {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

Runtime& rt() {
  static Runtime r;
  return r;
}

struct Buffer {
  void* ptr;
  size_t bytes;
};

static std::unordered_map<wgpt_buf, Buffer>& registry() {
  static std::unordered_map<wgpt_buf, Buffer> m;
  return m;
}
static wgpt_buf g_next_handle = 1;

void* resolve(wgpt_buf h, size_t need, const char* what) {
  auto it = registry().find(h);
  if (it == registry().end()) {
    fail(WGPT_ERR_ARG, "%s: unknown buffer handle %llu", what, (unsigned long long)h);
    return nullptr;
  }
  if (it->second.bytes < need) {
    fail(WGPT_ERR_ARG, "%s: buffer holds %zu bytes, %zu needed", what, it->second.bytes, need);
    return nullptr;
  }
  return it->second.ptr;
}

}  // namespace wgpt

using namespace wgpt;

// Splits [0, count) over up to 16 host threads.
template <typename F>
static void parallel_for(size_t count, F fn) {
  size_t nt = std::min<size_t>(std::max(1u, std::thread::hardware_concurrency()), 16);
  if (count < (1u << 16)) nt = 1;
  if (nt == 1) {
    fn(0, count);
    return;
  }
  std::vector<std::thread> th;
  const size_t step = (count + nt - 1) / nt;
  for (size_t t = 0; t < nt; ++t) {
    const size_t lo = t * step, hi = std::min(count, lo + step);
    if (lo < hi) th.emplace_back([=] { fn(lo, hi); });
  }
  for (auto& t : th) t.join();
}

extern "C" {

const char* wgpt_last_error(void) { return g_err; }

int wgpt_init(int device) {
  Runtime& r = rt();
  if (r.ready) {
    if (r.device == device) return WGPT_OK;
    return fail(WGPT_ERR_STATE, "already initialised on device %d", r.device);
  }
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0)
    return fail(WGPT_ERR_HIP, "no HIP device available (%s); this library has no CPU fallback",
                e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
  if (device < 0 || device >= count) return fail(WGPT_ERR_ARG, "device %d out of range (%d devices)", device, count);
  WGPT_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  WGPT_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(WGPT_ERR_STATE, "device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
  r.compute_units = prop.multiProcessorCount;
  {
    const int rc = setup_noalloc_scratch(device);
    if (rc) return rc;
  }
  WGPT_HIP(hipStreamCreateWithFlags(&r.stream, hipStreamNonBlocking));
  r.device = device;
  r.ready = true;
  return WGPT_OK;
}

int wgpt_shutdown(void) {
  Runtime& r = rt();
  if (!r.ready) return WGPT_OK;
  WGPT_HIP(hipStreamSynchronize(r.stream));
  destroy_all_models();
  for (auto& kv : registry()) (void)hipFree(kv.second.ptr);
  registry().clear();
  release_scratch();
  WGPT_HIP(hipStreamDestroy(r.stream));
  r.stream = nullptr;
  r.ready = false;
  r.device = -1;
  return WGPT_OK;
}

int wgpt_device_info(char* name, size_t name_len, int* compute_units, uint64_t* hbm_bytes) {
  WGPT_REQUIRE_INIT();
  hipDeviceProp_t prop;
  WGPT_HIP(hipGetDeviceProperties(&prop, rt().device));
  if (name && name_len) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (hbm_bytes) *hbm_bytes = (uint64_t)prop.totalGlobalMem;
  return WGPT_OK;
}

int wgpt_alloc(size_t bytes, wgpt_buf* out) {
  WGPT_REQUIRE_INIT();
  if (!out) return fail(WGPT_ERR_ARG, "wgpt_alloc: out is NULL");
  if (bytes == 0) return fail(WGPT_ERR_ARG, "wgpt_alloc: zero-sized buffer");
  void* p = nullptr;
  // 16 bytes of slack so that a float4 access to the last elements of a buffer whose
  // element count is a multiple of 4 never leaves the allocation.
  hipError_t e = hipMalloc(&p, bytes + 16);
  if (e != hipSuccess) return fail(WGPT_ERR_NOMEM, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
  wgpt_buf h = g_next_handle++;
  registry()[h] = Buffer{p, bytes};
  *out = h;
  return WGPT_OK;
}

int wgpt_free(wgpt_buf buf) {
  WGPT_REQUIRE_INIT();
  auto it = registry().find(buf);
  if (it == registry().end()) return fail(WGPT_ERR_ARG, "wgpt_free: unknown buffer handle %llu", (unsigned long long)buf);
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  WGPT_HIP(hipFree(it->second.ptr));
  registry().erase(it);
  return WGPT_OK;
}

int wgpt_buf_size(wgpt_buf buf, size_t* bytes) {
  auto it = registry().find(buf);
  if (it == registry().end()) return fail(WGPT_ERR_ARG, "wgpt_buf_size: unknown buffer handle %llu", (unsigned long long)buf);
  if (bytes) *bytes = it->second.bytes;
  return WGPT_OK;
}

static int check_range(wgpt_buf h, size_t off, size_t n, const char* what, char** base) {
  if (off + n < off) return fail(WGPT_ERR_ARG, "%s: offset overflow", what);
  void* p = resolve(h, off + n, what);
  if (!p) return WGPT_ERR_ARG;
  *base = (char*)p + off;
  return WGPT_OK;
}

int wgpt_upload(wgpt_buf dst, size_t dst_off, const void* src, size_t bytes) {
  WGPT_REQUIRE_INIT();
  if (bytes == 0) return WGPT_OK;
  if (!src) return fail(WGPT_ERR_ARG, "wgpt_upload: src is NULL");
  char* d;
  int rc = check_range(dst, dst_off, bytes, "wgpt_upload", &d);
  if (rc) return rc;
  WGPT_HIP(hipMemcpyAsync(d, src, bytes, hipMemcpyHostToDevice, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  return WGPT_OK;
}

int wgpt_download(void* dst, wgpt_buf src, size_t src_off, size_t bytes) {
  WGPT_REQUIRE_INIT();
  if (bytes == 0) return WGPT_OK;
  if (!dst) return fail(WGPT_ERR_ARG, "wgpt_download: dst is NULL");
  char* s;
  int rc = check_range(src, src_off, bytes, "wgpt_download", &s);
  if (rc) return rc;
  WGPT_HIP(hipMemcpyAsync(dst, s, bytes, hipMemcpyDeviceToHost, rt().stream));
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  return WGPT_OK;
}

int wgpt_copy(wgpt_buf dst, size_t dst_off, wgpt_buf src, size_t src_off, size_t bytes) {
  WGPT_REQUIRE_INIT();
  if (bytes == 0) return WGPT_OK;
  char *d, *s;
  int rc = check_range(dst, dst_off, bytes, "wgpt_copy(dst)", &d);
  if (rc) return rc;
  rc = check_range(src, src_off, bytes, "wgpt_copy(src)", &s);
  if (rc) return rc;
  WGPT_HIP(hipMemcpyAsync(d, s, bytes, hipMemcpyDeviceToDevice, rt().stream));
  return WGPT_OK;
}

int wgpt_sync(void) {
  WGPT_REQUIRE_INIT();
  WGPT_HIP(hipStreamSynchronize(rt().stream));
  return WGPT_OK;
}

// ---- synthetic tensors (host only) ----

void wgpt_synth_normal(uint32_t seed, uint32_t tensor_id, size_t count, double std_, float* out) {
  const uint32_t key = wgpt_tensor_key(seed, tensor_id);
  parallel_for(count, [=](size_t lo, size_t hi) {
    for (size_t i = lo; i < hi; ++i) out[i] = wgpt_synth_normal_at(key, (uint32_t)i, std_);
  });
}

void wgpt_synth_tokens(uint32_t seed, uint32_t tensor_id, size_t count, uint32_t vocab, int32_t* out) {
  const uint32_t key = wgpt_tensor_key(seed, tensor_id);
  for (size_t i = 0; i < count; ++i) out[i] = wgpt_synth_token_at(key, (uint32_t)i, vocab);
}

void wgpt_synth_int8_packed(uint32_t seed, uint32_t tensor_id, size_t K, size_t N, int32_t* out) {
  const uint32_t key = wgpt_tensor_key(seed, tensor_id);
  const size_t words = K * (N / 4);
  parallel_for(words, [=](size_t lo, size_t hi) {
    for (size_t w = lo; w < hi; ++w) {
      uint32_t word = 0;
      for (uint32_t e = 0; e < 4; ++e) {
        const int32_t q = wgpt_synth_int8_at(key, (uint32_t)(w * 4 + e));
        word |= ((uint32_t)q & 0xffu) << (8 * e);
      }
      out[w] = (int32_t)word;
    }
  });
}

void wgpt_synth_uniform(uint32_t seed, uint32_t tensor_id, size_t count, double lo, double hi, float* out) {
  const uint32_t key = wgpt_tensor_key(seed, tensor_id);
  for (size_t i = 0; i < count; ++i) out[i] = wgpt_synth_uniform_at(key, (uint32_t)i, lo, hi);
}

uint32_t wgpt_synth_tensor_id(const char* name) {
  uint32_t h = 2166136261u;
  for (const unsigned char* p = (const unsigned char*)name; *p; ++p) {
    h ^= *p;
    h *= 16777619u;
  }
  return h;
}

}  // extern "C"
