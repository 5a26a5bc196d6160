// Fused multi-head attention forward (flash attention) for bf16 / fp16:
//     O = softmax(scale * Q K^T + bias + mask) V,   optional LSE = m + log l.
//
// One work-group = 128 query rows of one (batch, head) unit, 4 waves x 32 rows.  Keys
// are walked in blocks of 64.  Both products are issued transposed so that a lane owns
// ONE query row for the whole kernel:
//   S^T = K Q^T : A operand = K fragment (rows = keys), B operand = Q fragment kept in
//                 registers; the 32x32 accumulator layout puts query l%32 in lane l and
//                 keys in the lane's registers, so row max / row sum are plain register
//                 reductions plus one exchange with lane l^32 (which holds the other keys).
//   O^T += V^T P^T : P stays in registers (the accumulator registers, converted, ARE
//                 the B operand); V is staged untransposed [key][h] and read with the LDS
//                 transpose loads, which deliver four consecutive keys of one h.
// Online softmax in the exp2 domain (scale * log2 e folded into one multiply), running
// max m and per-lane partial sum l; O is rescaled by 2^(m_old - m_new) per block and
// divided by l once at the end.  Causal: key > query masked (top-left aligned), key
// blocks past the diagonal are never visited, work-groups are issued heaviest first.
#include <utility>

#include "common.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int BR = 128;  // query rows per work-group
constexpr int BC = 64;   // keys per step
constexpr int NT = 256;
constexpr uint32_t kOob = 0x80000000u;
constexpr float kLog2e = 1.4426950408889634f;

struct FmhaParams {
  const void* q;
  const void* k;
  const void* v;
  const void* bias;
  void* out;
  float* lse;
  int H, F, T;
  int nqb;       // query blocks per unit
  float scale2;  // head_scale * log2(e)
};

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(static_cast<F&&>(f), std::make_integer_sequence<int, N>{});
}

template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  typedef bf16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <> struct Elem<_Float16> {
  typedef f16x8 vec8;
  static __device__ __forceinline__ floatx16 mfma(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ floatx16 zero16() {
  return floatx16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ u32x4 buf_load(__amdgpu_buffer_rsrc_t r, uint32_t voff) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
}

// T: element type; HP: head size padded to 64 / 128 / 256.
template <typename T, int HP, bool CAUSAL, bool BIAS>
__global__ __launch_bounds__(NT, (HP <= 128 ? 2 : 1)) void fmha_fwd_kernel(FmhaParams p) {
  typedef typename Elem<T>::vec8 V8;
  constexpr int KCH = HP / 8;              // 16-byte chunks per K/V row
  constexpr int NCH = BC * KCH / NT;       // chunks per thread per tile
  constexpr int K_ROW = HP * 2;            // K tile row, bytes (chunks XOR-swizzled by row)
  constexpr int V_ROW = HP * 2 + 64;       // V tile row, bytes (padded)
  constexpr int K_BYTES = BC * K_ROW, V_BYTES = BC * V_ROW;
  constexpr int STAGE = K_BYTES + V_BYTES;
  constexpr int KS = HP / 16;              // k-steps of the S product
  constexpr int HT = HP / 32;              // 32-wide h tiles of O
  __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5, l32 = lane & 31;
  const int unit = blockIdx.x / p.nqb;
  const int qb = p.nqb - 1 - blockIdx.x % p.nqb;  // heaviest (latest) query blocks first
  const int q0 = qb * BR;
  const int H = p.H, F = p.F, Tk = p.T;

  const T* Q = reinterpret_cast<const T*>(p.q) + (int64_t)unit * F * H;
  const T* K = reinterpret_cast<const T*>(p.k) + (int64_t)unit * Tk * H;
  const T* V = reinterpret_cast<const T*>(p.v) + (int64_t)unit * Tk * H;

  // ---- Q fragments (B operand of S^T): lane holds query row `qrow`, h = 16 s + 8 g .. +7.
  const int qrow = q0 + wave * 32 + l32;
  V8 qf[KS];
  {
    const int rows_left = F - q0;  // > 0
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(Q + (int64_t)q0 * H, (uint32_t)rows_left * H * 2);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const int h = 16 * s + 8 * g;
      const uint32_t off = h < H ? (uint32_t)(((wave * 32 + l32) * H + h) * 2) : kOob;
      qf[s] = __builtin_bit_cast(V8, buf_load(rq, off));
    }
  }

  // ---- staging of K / V tiles: chunk ch = tid + i NT -> key row ch / KCH, chunk ch % KCH.
  uint32_t voff[NCH];
  int koff[NCH], vlds[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int ch = tid + i * NT;
    const int row = ch / KCH, c = ch % KCH;
    voff[i] = c * 8 < H ? (uint32_t)((row * H + c * 8) * 2) : kOob;
    koff[i] = row * K_ROW + ((c ^ (row & 7)) << 4);
    vlds[i] = row * V_ROW + (c << 4);
  }
  u32x4 kr[NCH], vr[NCH];
  auto load_tiles = [&](int t0) {
    const uint32_t bytes = (uint32_t)(Tk - t0) * H * 2;  // rows past T read as zero
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(K + (int64_t)t0 * H, bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(V + (int64_t)t0 * H, bytes);
#pragma unroll
    for (int i = 0; i < NCH; ++i) kr[i] = buf_load(rk, voff[i]);
#pragma unroll
    for (int i = 0; i < NCH; ++i) vr[i] = buf_load(rv, voff[i]);
  };
  auto store_tiles = [&](char* stage) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) *reinterpret_cast<u32x4*>(stage + koff[i]) = kr[i];
#pragma unroll
    for (int i = 0; i < NCH; ++i) *reinterpret_cast<u32x4*>(stage + K_BYTES + vlds[i]) = vr[i];
  };

  floatx16 ot[HT];
#pragma unroll
  for (int i = 0; i < HT; ++i) ot[i] = zero16();
  float m_run = -INFINITY, l_run = 0.0f;

  const int kend = CAUSAL ? min(Tk, q0 + BR) : Tk;  // keys this work-group can see
  const int nblk = (kend + BC - 1) / BC;
  const int wq_min = q0 + wave * 32, wq_max = wq_min + 31;

  load_tiles(0);
  store_tiles(lds);
  __syncthreads();

  for (int it = 0; it < nblk; ++it) {
    const int t0 = it * BC;
    const char* ks_ = lds + (it & 1) * STAGE;
    const char* vs_ = ks_ + K_BYTES;
    const bool more = it + 1 < nblk;
    if (more) load_tiles(t0 + BC);

    if (!CAUSAL || t0 <= wq_max) {  // wave-uniform: this wave has at least one visible key
      // ---- S^T = K Q^T, two 32-key tiles
      floatx16 st[2];
      st[0] = zero16();
      st[1] = zero16();
#pragma unroll
      for (int s = 0; s < KS; ++s) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
          const int row = kt * 32 + l32;
          const int c = 2 * s + g;
          const u32x4 kv =
              *reinterpret_cast<const u32x4*>(ks_ + row * K_ROW + ((c ^ (row & 7)) << 4));
          st[kt] = Elem<T>::mfma(__builtin_bit_cast(V8, kv), qf[s], st[kt]);
        }
      }
      // ---- scale (+ bias), masks.  st[kt][i] <-> key t0 + 32 kt + 8 (i/4) + 4 g + i%4.
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) st[kt][i] *= p.scale2;
      if constexpr (BIAS) {
        if (qrow < F) {
          const T* bp = reinterpret_cast<const T*>(p.bias) + ((int64_t)unit * F + qrow) * Tk;
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int key = t0 + 32 * kt + 8 * (i / 4) + 4 * g + (i % 4);
              if (key < Tk) st[kt][i] += kLog2e * (float)bp[key];
            }
        }
      }
      const bool diag = CAUSAL && (t0 + BC - 1 > wq_min);
      const bool tail = t0 + BC > Tk;
      if (diag || tail) {
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = t0 + 32 * kt + 8 * (i / 4) + 4 * g + (i % 4);
            if ((CAUSAL && key > qrow) || key >= Tk) st[kt][i] = -INFINITY;
          }
      }
      // ---- online softmax for this lane's query row
      float mx = st[0][0];
#pragma unroll
      for (int i = 1; i < 16; ++i) mx = fmaxf(mx, st[0][i]);
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, st[1][i]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // first block: exp2(-inf) = 0
      float rs = 0.0f;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          st[kt][i] = __builtin_amdgcn_exp2f(st[kt][i] - m_new);
          rs += st[kt][i];
        }
      l_run = l_run * alpha + rs;
      m_run = m_new;
#pragma unroll
      for (int ht = 0; ht < HT; ++ht)
#pragma unroll
        for (int i = 0; i < 16; ++i) ot[ht][i] *= alpha;
      // ---- O^T += V^T P^T.  MFMA (kt, hf) contracts keys 32 kt + 16 hf + {0..3, 8..11} + 4 g.
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          V8 pf;
#pragma unroll
          for (int j = 0; j < 8; ++j) pf[j] = (T)st[kt][8 * hf + j];
          const int pl = lane & 15;
          const int kb = 32 * kt + 16 * hf + 4 * g;
#pragma unroll
          for (int ht = 0; ht < HT; ++ht) {
            const int cb = 32 * ht + ((lane >> 4) & 1) * 16;
            const char* a0 = vs_ + (kb + (pl >> 2)) * V_ROW + (cb + 4 * (pl & 3)) * 2;
            typedef short4v __attribute__((address_space(3))) * lds_ptr;
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(a0));
            const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(a0 + 8 * V_ROW));
            u32x4 vv;
            vv[0] = __builtin_bit_cast(u32x2, lo)[0];
            vv[1] = __builtin_bit_cast(u32x2, lo)[1];
            vv[2] = __builtin_bit_cast(u32x2, hi)[0];
            vv[3] = __builtin_bit_cast(u32x2, hi)[1];
            ot[ht] = Elem<T>::mfma(__builtin_bit_cast(V8, vv), pf, ot[ht]);
          }
        }
      }
    }

    if (more) store_tiles(lds + ((it + 1) & 1) * STAGE);
    __syncthreads();
  }

  // ---- finish: l = both halves' partial sums; O = O^T / l; LSE = m ln2 + ln l.
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  if (qrow < F) {
    T* orow = reinterpret_cast<T*>(p.out) + ((int64_t)unit * F + qrow) * H;
    static_for<HT>([&](auto HTI) {
      constexpr int ht = decltype(HTI)::value;
      const floatx16 t = ot[ht];
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int h = 32 * ht + 8 * qd + 4 * g;
        if (h < H) {  // H % 8 == 0, so the four values are all in range
          union { T e[4]; u32x2 w; } o;
          o.e[0] = (T)(t[4 * qd + 0] * inv);
          o.e[1] = (T)(t[4 * qd + 1] * inv);
          o.e[2] = (T)(t[4 * qd + 2] * inv);
          o.e[3] = (T)(t[4 * qd + 3] * inv);
          *reinterpret_cast<u32x2*>(orow + h) = o.w;
        }
      }
    });
    if (p.lse && g == 0) p.lse[(int64_t)unit * F + qrow] = m_run * 0.6931471805599453f + logf(l_tot);
  }
}

template <typename T, int HP>
void launch_hp(const FmhaParams& p, int units, bool causal, bool bias, hipStream_t st) {
  const dim3 grid((unsigned)(units * p.nqb)), block(NT);
  if (causal) {
    if (bias) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, true, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, true, false>), grid, block, 0, st, p);
  } else {
    if (bias) hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, false, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((fmha_fwd_kernel<T, HP, false, false>), grid, block, 0, st, p);
  }
}

template <typename T>
void launch_t(const FmhaParams& p, int units, bool causal, bool bias, hipStream_t st) {
  // Head-size classes of the reference's policy choice (fmha_forward.h:622-646).
  if (p.H <= 64) launch_hp<T, 64>(p, units, causal, bias, st);
  else if (p.H <= 128) launch_hp<T, 128>(p, units, causal, bias, st);
  else launch_hp<T, 256>(p, units, causal, bias, st);
}

}  // namespace

extern "C" int xmk_fmha_fwd(const void* query, const void* key, const void* value, const void* bias,
                            void* out, float* lse, int32_t dtype, uint32_t num_batches,
                            uint32_t num_heads, uint32_t head_size, uint32_t num_queries,
                            uint32_t num_keys, float head_scale, int32_t causal, void* stream) {
  if (!query || !key || !value || !out) return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: null pointer");
  if (dtype != XMK_F16 && dtype != XMK_BF16)
    return xmk::fail(XMK_INTERNAL, "Invalid MHA datatype");  // xetla_gpu_fused_mha_runner.cc:145
  if (num_batches == 0 || num_heads == 0 || head_size == 0 || num_queries == 0 || num_keys == 0)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: empty dimension");
  if (head_size > 256)
    return xmk::fail(XMK_UNIMPLEMENTED, "fmha_fwd: head_size %u > 256 (fmha_forward.h:642)", head_size);
  if (head_size % 8 != 0)
    return xmk::fail(XMK_UNIMPLEMENTED, "fmha_fwd: head_size %u is not a multiple of 8", head_size);
  const uint64_t units = (uint64_t)num_batches * num_heads;
  const uint64_t nqb = (num_queries + BR - 1) / BR;
  if (units * nqb > 0x7fffffffull || (uint64_t)num_keys * head_size * 2 >= kOob ||
      (uint64_t)num_queries * head_size * 2 >= kOob)
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: shape too large");
  if (!xmk::aligned(query, 16) || !xmk::aligned(key, 16) || !xmk::aligned(value, 16) ||
      !xmk::aligned(out, 16))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fmha_fwd: tensors must be 16-byte aligned");
  FmhaParams p;
  p.q = query; p.k = key; p.v = value; p.bias = bias; p.out = out; p.lse = lse;
  p.H = (int)head_size; p.F = (int)num_queries; p.T = (int)num_keys;
  p.nqb = (int)nqb;
  p.scale2 = head_scale * kLog2e;
  xmk::trace("fmha_fwd B=%u N=%u F=%u T=%u H=%u causal=%d bias=%d lse=%d", num_batches, num_heads,
             num_queries, num_keys, head_size, causal, bias != nullptr, lse != nullptr);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == XMK_BF16) launch_t<__bf16>(p, (int)units, causal != 0, bias != nullptr, st);
  else launch_t<_Float16>(p, (int)units, causal != 0, bias != nullptr, st);
  return xmk::check_launch("fmha_fwd");
}
