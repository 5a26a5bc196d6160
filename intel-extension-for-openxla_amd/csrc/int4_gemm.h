// Internal interface of the int4 weight-only GEMM: the public entry point plus the fused
// epilogue the decode step uses.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace xmk {

// out = fp16( gelu?(acc + bias) + add0 + add1 );  add0 / add1: optional fp16 [M, N] addends.
struct Int4Epilogue {
  int gelu = 0;
  const void* add0 = nullptr;
  const void* add1 = nullptr;
};

int int4_gemm_launch(const void* act, const void* qweight, const void* scales, const void* zeros,
                     const void* bias, void* out, int64_t m, int64_t k, int64_t n, int64_t group,
                     const Int4Epilogue& ep, hipStream_t st);

}  // namespace xmk
