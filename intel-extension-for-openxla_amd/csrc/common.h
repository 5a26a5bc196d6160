// Shared host-side helpers of the kernel library: status codes, the
// thread-local error message, and launch checking.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "xmk.h"

namespace xmk {

// Records `fmt...` as the calling thread's last error and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Non-zero when XMK_TRACE is set: entry points then print one line per call
// (target, shapes, chosen tile) to stderr, like the reference's VLOG(1) lines
// (onednn_matmul_utils.cc:502,506; xetla_gpu_fused_mha_runner.cc:58-111).
bool trace_enabled();
void trace(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(XMK_INTERNAL, "%s: launch failed: %s", what, hipGetErrorString(e));
  return XMK_OK;
}

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace xmk
