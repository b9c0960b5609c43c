// Shared host-side plumbing of the library: error reporting, the device buffer
// registry behind wgpt_buf handles, and the single HIP stream everything runs on.
#ifndef WGPT_COMMON_H
#define WGPT_COMMON_H

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>

#include "../../include/webgpt_amd.h"

namespace wgpt {

// Records the message returned by wgpt_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

struct Runtime {
  bool ready = false;
  int device = -1;
  int compute_units = 0;
  hipStream_t stream = nullptr;
};
Runtime& rt();

// Resolves a handle to its device pointer after checking that the buffer holds at
// least `need` bytes. Returns nullptr (and records the error) otherwise.
void* resolve(wgpt_buf h, size_t need, const char* what);

// Frees the grow-only scratch buffers of the block entry points.
void release_scratch();
// Looks up this device's address of the fixed workspace of wgpt_matmul_bias_noalloc; called by wgpt_init
// with `device` current.
int setup_noalloc_scratch(int device);

#define WGPT_HIP(call)                                                                      \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) return ::wgpt::fail(WGPT_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_)); \
  } while (0)

#define WGPT_REQUIRE_INIT()                                                                  \
  do {                                                                                      \
    if (!::wgpt::rt().ready) return ::wgpt::fail(WGPT_ERR_STATE, "wgpt_init() has not succeeded"); \
  } while (0)

}  // namespace wgpt

#endif
