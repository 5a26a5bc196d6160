// Device-wide MFMA rate probe: a loop of independent MFMA instructions and nothing else.
#include <hip/hip_runtime.h>

#include "common.h"
#include "xmk_probe.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kBlocks = 1024, kThreads = 256;

__device__ __forceinline__ floatx16 mma32(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mma32(f16x8 a, f16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx4 mma16(bf16x8 a, bf16x8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx4 mma16(f16x8 a, f16x8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// Operands: pseudo-random bit patterns (random sign and mantissa, exponent spread over 2^-7 .. 1),
// a hash of the lane and the register index, so that the data toggles as real matrices do.  The
// rate depends on it: constant or few-bit operands draw less power and run at a higher clock.
template <typename E, typename V8>
__device__ __forceinline__ V8 operand(uint32_t seed) {
  constexpr bool kBf16 = sizeof(V8) == 16 && __is_same(E, __bf16);
  V8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t h = (seed * 8u + j + 1u) * 2654435761u;
    h ^= h >> 15;
    h *= 2246822519u;
    h ^= h >> 13;
    const uint16_t bits = kBf16 ? (uint16_t)(((h >> 16) & 0x8000u) | ((120u + ((h >> 8) & 7u)) << 7) | (h & 0x7fu))
                                : (uint16_t)(((h >> 16) & 0x8000u) | ((8u + ((h >> 10) & 7u)) << 10) | (h & 0x3ffu));
    v[j] = __builtin_bit_cast(E, bits);
  }
  return v;
}

typedef int intx8 __attribute__((ext_vector_type(8)));

// fp8 (e4m3) operands: 32 bytes per lane; any byte but the two NaN encodings (0x7f, 0xff).
__device__ __forceinline__ intx8 operand_fp8(uint32_t seed) {
  intx8 v;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t h = (seed * 8u + j + 1u) * 2654435761u;
    h ^= h >> 15;
    h *= 2246822519u;
    h ^= h >> 13;
    v[j] = (int)(h & 0xbfbfbfbfu);  // exponent field below all-ones: finite values only
  }
  return v;
}

template <int TILE>
__global__ __launch_bounds__(kThreads) void mfma_rate_fp8_kernel(float* sink, int iters) {
  intx8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operand_fp8(threadIdx.x * 4 + i);
    b[i] = operand_fp8(threadIdx.x * 4 + i + 4096);
  }
  float s = 0.f;
  if constexpr (TILE == 32) {
    floatx16 acc[4][4] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[j], acc[i][j], 0, 0, 0, 127, 0, 127);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  } else {
    floatx4 acc[8][8] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[i & 3], b[j & 3], acc[i][j], 0, 0, 0, 127, 0, 127);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  }
  sink[blockIdx.x * kThreads + threadIdx.x] = s;
}

template <typename E, typename V8, int TILE>
__global__ __launch_bounds__(kThreads) void mfma_rate_kernel(float* sink, int iters) {
  V8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operand<E, V8>(threadIdx.x * 4 + i);
    b[i] = operand<E, V8>(threadIdx.x * 4 + i + 4096);
  }
  float s = 0.f;
  if constexpr (TILE == 32) {
    floatx16 acc[4][4] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = mma32(a[i], b[j], acc[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[i][j][e];
  } else {
    floatx4 acc[8][8] = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = mma16(a[i & 3], b[j & 3], acc[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) s += acc[i][j][e];
  }
  sink[blockIdx.x * kThreads + threadIdx.x] = s;
}

}  // namespace

extern "C" double xmk_probe_mfma_flops(int32_t dtype, int32_t tile, int32_t iters) {
  const double k = (tile == 32 ? 16.0 : 32.0) * (dtype == XMK_F8E4M3FN ? 4.0 : 1.0);  // depth of one MFMA
  const double per_round = (tile == 32 ? 16.0 : 64.0) * 2.0 * tile * tile * k;
  return per_round * iters * kBlocks * (kThreads / 64);
}

extern "C" int xmk_probe_mfma_rate(int32_t dtype, int32_t tile, int32_t iters, void* sink, uint64_t sink_bytes,
                                   void* stream) {
  if (!sink || sink_bytes < (uint64_t)kBlocks * kThreads * sizeof(float))
    return xmk::fail(XMK_INVALID_ARGUMENT, "probe_mfma_rate: sink must hold %d floats", kBlocks * kThreads);
  if ((tile != 32 && tile != 16) || iters <= 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "probe_mfma_rate: tile must be 32 or 16, iters positive");
  if (dtype != XMK_BF16 && dtype != XMK_F16 && dtype != XMK_F8E4M3FN)
    return xmk::fail(XMK_INVALID_ARGUMENT, "probe_mfma_rate: dtype must be bf16, f16 or f8e4m3fn");
  hipStream_t st = (hipStream_t)stream;
  float* out = static_cast<float*>(sink);
  const dim3 grid(kBlocks), block(kThreads);
  if (dtype == XMK_BF16) {
    if (tile == 32) hipLaunchKernelGGL((mfma_rate_kernel<__bf16, bf16x8, 32>), grid, block, 0, st, out, iters);
    else hipLaunchKernelGGL((mfma_rate_kernel<__bf16, bf16x8, 16>), grid, block, 0, st, out, iters);
  } else if (dtype == XMK_F8E4M3FN) {
    if (tile == 32) hipLaunchKernelGGL((mfma_rate_fp8_kernel<32>), grid, block, 0, st, out, iters);
    else hipLaunchKernelGGL((mfma_rate_fp8_kernel<16>), grid, block, 0, st, out, iters);
  } else {
    if (tile == 32) hipLaunchKernelGGL((mfma_rate_kernel<_Float16, f16x8, 32>), grid, block, 0, st, out, iters);
    else hipLaunchKernelGGL((mfma_rate_kernel<_Float16, f16x8, 16>), grid, block, 0, st, out, iters);
  }
  return xmk::check_launch("probe_mfma_rate");
}
