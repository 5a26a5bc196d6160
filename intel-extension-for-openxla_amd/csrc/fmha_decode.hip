// Attention for a single query row per (batch, head) unit (decode, seq_q = 1): HBM-bound
// streaming of the K and V cache rows.
//
// The keys of a unit are split over `splits` work-groups so that a few dozen units still
// fill 256 CUs (flash-decoding).  Pass 1 (fmha_decode_split_kernel): a work-group takes
// one contiguous chunk of keys; lanes run along h (16 bytes each, a row is read as one
// contiguous segment), scores are reduced across the lanes of a row with DPP/permute
// shuffles, the chunk's softmax statistics are formed in LDS and the chunk's unnormalised
// output  sum_t 2^(s_t - m) V[t,:]  is written to the workspace together with (m, l).
// Pass 2 (fmha_decode_merge_kernel): one work-group per unit rescales and adds the
// partial results and writes the output row.
#include <cstdlib>

#include <algorithm>
#include <atomic>

#include "common.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr float kLog2e = 1.4426950408889634f;
constexpr int NT = 256;

struct DecodeParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* ws;  // [units][splits][H + 2]: partial O (H floats), m, l
  int N, H, T;
  int64_t kv_head_stride;  // elements between consecutive heads' caches
  int splits, chunk;
  float scale2;
};

template <typename T>
__device__ __forceinline__ void unpack8(u32x4 raw, float* f) {
  union { u32x4 u; T e[8]; } x;
  x.u = raw;
#pragma unroll
  for (int i = 0; i < 8; ++i) f[i] = (float)x.e[i];
}

// LPR: lanes per row (H <= 8 * LPR), a power of two <= 32.
template <typename T, int LPR>
__global__ __launch_bounds__(NT) void fmha_decode_split_kernel(DecodeParams p) {
  constexpr int RPP = NT / LPR;  // rows per pass of the block
  constexpr int MAXCH = 512;     // keys per chunk, upper bound
  __shared__ float s_score[MAXCH];
  __shared__ float s_red[NT / 64][8 * 32];  // per-wave partial outputs (up to 256 h)
  __shared__ float s_stat[2];

  const int tid = threadIdx.x;
  const int unit = blockIdx.x / p.splits, split = blockIdx.x % p.splits;
  const int t_begin = split * p.chunk;
  const int t_end = min(p.T, t_begin + p.chunk);
  const int nkeys = t_end - t_begin;  // may be <= 0 for trailing splits
  const int H = p.H;
  const int lr = tid % LPR, rr = tid / LPR;
  const int h0 = lr * 8;
  const bool h_ok = h0 < H;

  const T* Q = reinterpret_cast<const T*>(p.q) + (int64_t)unit * H;
  const int64_t kv_base = (int64_t)(unit / p.N) * p.N * p.kv_head_stride + (int64_t)(unit % p.N) * p.kv_head_stride;
  const T* K = reinterpret_cast<const T*>(p.k) + kv_base;
  const T* V = reinterpret_cast<const T*>(p.v) + kv_base;
  float* wsu = p.ws + ((int64_t)unit * p.splits + split) * (H + 2);

  float qf[8];
  {
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (h_ok) raw = *reinterpret_cast<const u32x4*>(Q + h0);
    unpack8<T>(raw, qf);
#pragma unroll
    for (int i = 0; i < 8; ++i) qf[i] *= p.scale2;
  }

  // ---- scores s_t = scale2 * q . k_t
  for (int r0 = 0; r0 < nkeys; r0 += RPP * 4) {
    u32x4 raw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = r0 + j * RPP + rr;
      raw[j] = u32x4{0u, 0u, 0u, 0u};
      if (r < nkeys && h_ok) raw[j] = *reinterpret_cast<const u32x4*>(K + (int64_t)(t_begin + r) * H + h0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float kf[8];
      unpack8<T>(raw[j], kf);
      float d = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) d = fmaf(qf[i], kf[i], d);
#pragma unroll
      for (int o = LPR / 2; o >= 1; o >>= 1) d += __shfl_xor(d, o);
      const int r = r0 + j * RPP + rr;
      if (lr == 0 && r < nkeys) s_score[r] = d;
    }
  }
  __syncthreads();

  // ---- chunk statistics: m = max s, p_t = 2^(s_t - m), l = sum p_t   (wave 0)
  if (tid < 64) {
    float m = -INFINITY;
    for (int r = tid; r < nkeys; r += 64) m = fmaxf(m, s_score[r]);
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    float l = 0.f;
    for (int r = tid; r < nkeys; r += 64) {
      const float e = __builtin_amdgcn_exp2f(s_score[r] - m);
      s_score[r] = e;
      l += e;
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) l += __shfl_xor(l, o);
    if (tid == 0) { s_stat[0] = m; s_stat[1] = l; }
  }
  __syncthreads();

  // ---- partial output: acc[h] = sum_t p_t V[t, h]
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  for (int r0 = 0; r0 < nkeys; r0 += RPP * 4) {
    u32x4 raw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = r0 + j * RPP + rr;
      raw[j] = u32x4{0u, 0u, 0u, 0u};
      if (r < nkeys && h_ok) raw[j] = *reinterpret_cast<const u32x4*>(V + (int64_t)(t_begin + r) * H + h0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = r0 + j * RPP + rr;
      const float pt = r < nkeys ? s_score[r] : 0.f;
      float vf[8];
      unpack8<T>(raw[j], vf);
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = fmaf(pt, vf[i], acc[i]);
    }
  }
  // Rows of one wave that share h: lanes lr, lr + LPR, ... -> reduce inside the wave, then over waves.
#pragma unroll
  for (int o = 32; o >= LPR; o >>= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] += __shfl_xor(acc[i], o);
  const int wave = tid >> 6, lane = tid & 63;
  if (lane < LPR) {
#pragma unroll
    for (int i = 0; i < 8; ++i) s_red[wave][lane * 8 + i] = acc[i];
  }
  __syncthreads();
  for (int h = tid; h < H; h += NT) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) s += s_red[w][h];
    wsu[h] = s;
  }
  if (tid == 0) { wsu[H] = s_stat[0]; wsu[H + 1] = s_stat[1]; }
}

constexpr int MAXSPLITS = 1024;

// Block-wide max / sum of one float per thread (NT threads); every thread gets the result.
template <bool IS_MAX>
__device__ __forceinline__ float block_reduce(float v, float* s_tmp) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    const float w = __shfl_xor(v, o);
    v = IS_MAX ? fmaxf(v, w) : v + w;
  }
  __syncthreads();  // s_tmp may still be read from an earlier call
  if ((threadIdx.x & 63) == 0) s_tmp[threadIdx.x >> 6] = v;
  __syncthreads();
  v = s_tmp[0];
#pragma unroll
  for (int i = 1; i < NT / 64; ++i) v = IS_MAX ? fmaxf(v, s_tmp[i]) : v + s_tmp[i];
  return v;
}

// One work-group per unit: the weights 2^(m_s - m) / l of the splits are formed once in LDS
// (thread s handles split s), then thread h adds up column h of the partial outputs with
// independent, coalesced loads.
template <typename T>
__global__ __launch_bounds__(NT) void fmha_decode_merge_kernel(DecodeParams p) {
  __shared__ float s_w[MAXSPLITS];
  __shared__ float s_tmp[NT / 64];
  const int unit = blockIdx.x, H = p.H, S = p.splits;
  const int64_t stride = H + 2;
  const float* wsu = p.ws + (int64_t)unit * S * stride;
  float m = -INFINITY;
  for (int s = threadIdx.x; s < S; s += NT) {
    const float ms = wsu[s * stride + H];
    s_w[s] = ms;
    m = fmaxf(m, ms);
  }
  m = block_reduce<true>(m, s_tmp);
  float l = 0.f;
  for (int s = threadIdx.x; s < S; s += NT) {
    const float ms = s_w[s];  // written by this thread
    const float w = ms > -INFINITY ? __builtin_amdgcn_exp2f(ms - m) : 0.f;
    l += wsu[s * stride + H + 1] * w;
    s_w[s] = w;
  }
  l = block_reduce<false>(l, s_tmp);  // its barriers also publish s_w
  const float inv = 1.0f / l;
  T* out = reinterpret_cast<T*>(p.out) + (int64_t)unit * H;
  for (int h = threadIdx.x; h < H; h += NT) {
    float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;
    int s = 0;
    for (; s + 4 <= S; s += 4) {
      o0 += wsu[(s + 0) * stride + h] * s_w[s + 0];
      o1 += wsu[(s + 1) * stride + h] * s_w[s + 1];
      o2 += wsu[(s + 2) * stride + h] * s_w[s + 2];
      o3 += wsu[(s + 3) * stride + h] * s_w[s + 3];
    }
    for (; s < S; ++s) o0 += wsu[s * stride + h] * s_w[s];
    out[h] = (T)(((o0 + o1) + (o2 + o3)) * inv);
  }
}

// Up to 16 splits (what 64 and more units plan): no LDS and no barrier.  Every thread loads all the
// splits' statistics (the same few cache lines for the whole work-group) and its own column of the partial
// outputs in one go, so the kernel costs one round of loads instead of three dependent ones.
constexpr int SMALL_SPLITS = 16;
template <typename T>
__global__ __launch_bounds__(NT) void fmha_decode_merge_small_kernel(DecodeParams p) {
  const int unit = blockIdx.x, H = p.H, S = p.splits;
  const int64_t stride = H + 2;
  const float* wsu = p.ws + (int64_t)unit * S * stride;
  const int h = threadIdx.x < H ? threadIdx.x : 0;
  float ms[SMALL_SPLITS], ls[SMALL_SPLITS], os[SMALL_SPLITS];
#pragma unroll
  for (int s = 0; s < SMALL_SPLITS; ++s) {
    const bool ok = s < S;
    ms[s] = ok ? wsu[s * stride + H] : -INFINITY;
    ls[s] = ok ? wsu[s * stride + H + 1] : 0.f;
    os[s] = ok ? wsu[s * stride + h] : 0.f;
  }
  float m = ms[0];
#pragma unroll
  for (int s = 1; s < SMALL_SPLITS; ++s) m = fmaxf(m, ms[s]);
  // The partial outputs are added as four interleaved partial sums, like the general kernel's; l is
  // added split by split (the general kernel reduces per-thread shares across the work-group) and the
  // result is divided by l (there: multiplied by 1 / l), so the two kernels may differ in the last
  // bit of the 16-bit result.
  float l = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < SMALL_SPLITS; ++s) {
    const float w = ms[s] > -INFINITY ? __builtin_amdgcn_exp2f(ms[s] - m) : 0.f;
    l += ls[s] * w;
    if (s < (S & ~3)) o[s & 3] += os[s] * w;
    else o[0] += os[s] * w;
  }
  if (threadIdx.x < H)
    reinterpret_cast<T*>(p.out)[(int64_t)unit * H + threadIdx.x] = (T)(((o[0] + o[1]) + (o[2] + o[3])) / l);
}

// Work-groups the split kernel aims to have in flight (XMK_DECODE_WGS overrides the 1024).
uint32_t plan_target() {
  static const int target = [] {
    const char* e = getenv("XMK_DECODE_WGS");
    const int v = e ? atoi(e) : 0;
    return v >= 64 && v <= 65536 ? v : 1024;
  }();
  return (uint32_t)target;
}

void plan(uint32_t units, uint32_t T, int* splits, int* chunk) {
  // About plan_target() work-groups in flight, at least 64 and at most 512 keys per chunk.
  const uint32_t target = plan_target();
  int s = (int)((target + units - 1) / units);
  int c = (int)((T + s - 1) / s);
  if (c < 64) c = 64;
  if (c > 512) c = 512;
  c = (c + 31) / 32 * 32;
  *chunk = c;
  *splits = (int)((T + c - 1) / c);
}

template <typename T>
void launch(const DecodeParams& p, int units, hipStream_t st) {
  const dim3 grid((unsigned)(units * p.splits)), block(NT);
  if (p.H <= 64) hipLaunchKernelGGL((fmha_decode_split_kernel<T, 8>), grid, block, 0, st, p);
  else if (p.H <= 128) hipLaunchKernelGGL((fmha_decode_split_kernel<T, 16>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((fmha_decode_split_kernel<T, 32>), grid, block, 0, st, p);
  // XMK_DECODE_MERGE_GENERAL (read at every call, so that a test can compare the two merge kernels on one
  // shape in one process) sends every shape to the general kernel.
  const char* general = getenv("XMK_DECODE_MERGE_GENERAL");
  if (p.splits <= SMALL_SPLITS && p.H <= NT && !(general && *general && *general != '0'))
    hipLaunchKernelGGL((fmha_decode_merge_small_kernel<T>), dim3((unsigned)units), block, 0, st, p);
  else
    hipLaunchKernelGGL((fmha_decode_merge_kernel<T>), dim3((unsigned)units), block, 0, st, p);
}

}  // namespace

extern "C" size_t xmk_fmha_decode_workspace_bytes(uint32_t num_batches, uint32_t num_heads,
                                                  uint32_t head_size, uint32_t num_keys) {
  int splits, chunk;
  const uint32_t units = num_batches * num_heads;
  if (units == 0 || num_keys == 0) return 0;
  plan(units, num_keys, &splits, &chunk);
  return (size_t)units * splits * (head_size + 2) * sizeof(float);
}

extern "C" size_t xmk_fmha_decode_cache_workspace_bytes(uint32_t num_batches, uint32_t num_heads,
                                                        uint32_t head_size, uint32_t cache_capacity) {
  // The split count is not monotonic in the number of keys (the chunk is rounded to 32 and clamped
  // to 64..512 keys), so a cache is sized for the largest count any fill level 1..capacity plans.
  // With s = plan()'s split target per unit: up to 64 s keys the chunk is 64 and the count
  // ceil(t / 64) <= s; up to 512 s keys the chunk is at least t / s, so the count stays <= s (and
  // t = 64 s reaches s); beyond, the chunk is 512 and the count ceil(t / 512) grows with t.
  const uint32_t units = num_batches * num_heads;
  if (units == 0 || cache_capacity == 0) return 0;
  const uint64_t s = (plan_target() + units - 1) / units, cap = cache_capacity;
  const uint64_t most = cap <= 512 * s ? std::min((cap + 63) / 64, s) : (cap + 511) / 512;
  return (size_t)units * most * (head_size + 2) * sizeof(float);
}

namespace {

int decode_checked(const void* query, const void* key, const void* value, void* out, int32_t dtype,
                   uint32_t num_batches, uint32_t num_heads, uint32_t head_size, uint32_t num_keys,
                   int64_t kv_head_stride, float head_scale, void* workspace, size_t workspace_bytes,
                   const char* what, void* stream) {
  if (!query || !key || !value || !out || !workspace)
    return xmk::fail(XMK_INVALID_ARGUMENT, "%s: null pointer", what);
  if (dtype != XMK_F16 && dtype != XMK_BF16) return xmk::fail(XMK_INTERNAL, "Invalid MHA datatype");
  if (num_batches == 0 || num_heads == 0 || head_size == 0 || num_keys == 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "%s: empty dimension", what);
  if (head_size > 256 || head_size % 8 != 0)
    return xmk::fail(XMK_UNIMPLEMENTED, "%s: head_size must be a multiple of 8, at most 256", what);
  if (kv_head_stride < (int64_t)num_keys * head_size || kv_head_stride % 8 != 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "%s: kv_head_stride too small or not a multiple of 8", what);
  if (!xmk::aligned(query, 16) || !xmk::aligned(key, 16) || !xmk::aligned(value, 16))
    return xmk::fail(XMK_INVALID_ARGUMENT, "%s: tensors must be 16-byte aligned", what);
  const size_t need = xmk_fmha_decode_workspace_bytes(num_batches, num_heads, head_size, num_keys);
  if (workspace_bytes < need)
    return xmk::fail(XMK_INVALID_ARGUMENT, "%s: workspace of %zu bytes, %zu needed", what, workspace_bytes, need);
  DecodeParams p;
  p.q = query; p.k = key; p.v = value; p.out = out; p.ws = (float*)workspace;
  p.N = (int)num_heads; p.H = (int)head_size; p.T = (int)num_keys;
  p.kv_head_stride = kv_head_stride;
  p.scale2 = head_scale * kLog2e;
  const uint32_t units = num_batches * num_heads;
  plan(units, num_keys, &p.splits, &p.chunk);
  if (p.splits > MAXSPLITS)
    return xmk::fail(XMK_UNIMPLEMENTED, "%s: %u keys need %d splits, more than %d", what, num_keys, p.splits,
                     MAXSPLITS);
  xmk::trace("%s B=%u N=%u T=%u H=%u splits=%d chunk=%d", what, num_batches, num_heads, num_keys,
             head_size, p.splits, p.chunk);
  if (dtype == XMK_BF16) launch<__bf16>(p, (int)units, (hipStream_t)stream);
  else launch<_Float16>(p, (int)units, (hipStream_t)stream);
  return xmk::check_launch(what);
}

}  // namespace

extern "C" int xmk_fmha_decode(const void* query, const void* key, const void* value, void* out,
                               int32_t dtype, uint32_t num_batches, uint32_t num_heads,
                               uint32_t head_size, uint32_t num_keys, int64_t kv_head_stride,
                               float head_scale, void* workspace, size_t workspace_bytes,
                               void* stream) {
  return decode_checked(query, key, value, out, dtype, num_batches, num_heads, head_size, num_keys,
                        kv_head_stride, head_scale, workspace, workspace_bytes, "fmha_decode", stream);
}

// ---- The entry point that allocates nothing -------------------------------------------------
// Same kernels as xmk_fmha_decode; the partial results of the key splits go to a device array that
// is part of the library's code object instead of caller memory.  Every GPU holds its own copy of
// the array, at its own address, from the first call on that GPU until the process ends.
namespace {

constexpr size_t kStaticScratchBytes = size_t{4} << 20;  // 4 MiB: config 5 (64 units, 16 splits, head size 256) needs 1.06 MB
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

constexpr int kMaxDevices = 64;
std::atomic<float*> scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU, once looked up

// Device address of this GPU's copy of `scratch`.  The array's name is a host-side stand-in, not a
// device address; the address comes from the runtime, once per device, with that device current.
int static_scratch(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return xmk::fail(XMK_INTERNAL, "fmha_decode_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return xmk::fail(XMK_INTERNAL, "fmha_decode_static: device index %d", dev);
  float* p = scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* addr = nullptr;
    e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !addr)
      return xmk::fail(XMK_INTERNAL, "fmha_decode_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    p = static_cast<float*>(addr);
    scratch_ptr[dev].store(p, std::memory_order_release);  // concurrent first calls store the same address
  }
  *out = p;
  return XMK_OK;
}

}  // namespace

extern "C" size_t xmk_fmha_decode_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int xmk_fmha_decode_static_init(void) {
  float* ws = nullptr;
  return static_scratch(&ws);
}

extern "C" int xmk_fmha_decode_static(const void* query, const void* key, const void* value, void* out,
                                      int32_t dtype, uint32_t num_batches, uint32_t num_heads,
                                      uint32_t head_size, uint32_t num_keys, int64_t kv_head_stride,
                                      float head_scale, void* stream) {
  const size_t need = xmk_fmha_decode_workspace_bytes(num_batches, num_heads, head_size, num_keys);
  if (need > kStaticScratchBytes)
    return xmk::fail(XMK_INVALID_ARGUMENT,
                     "fmha_decode_static: this shape needs %zu bytes of scratch, the built-in array holds %zu; "
                     "use xmk_fmha_decode with a workspace", need, kStaticScratchBytes);
  float* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc != XMK_OK) return rc;
  // Every partial result the merge kernel reads is written by the split kernel of the same call, so
  // nothing needs clearing between calls.
  return decode_checked(query, key, value, out, dtype, num_batches, num_heads, head_size, num_keys,
                        kv_head_stride, head_scale, ws, kStaticScratchBytes, "fmha_decode_static", stream);
}
