// s8 x s8 -> s32 GEMM on the matrix cores (v_mfma_i32_32x32x32_i8), any layout and alignment; alpha = 1,
// beta = 0, no epilogue (the int8 dtype triple of onednn_matmul_utils.cc:605-610).
//
// Same shape as the fp32 kernel (gemm_f32.hip): 256 threads = 4 waves in 2 x 2, tile 128 x 128 (64 x 64
// for small products) x 64 k, 4 LDS stages, both operands k-contiguous in LDS ([row][64 bytes],
// XOR-swizzled 16-byte chunks) whatever their storage.  A lane gathers one 16-byte chunk (16 consecutive
// k of one row or column) per operand half -- one aligned vector load, or 16 byte loads (k-contiguous but
// unaligned, or [K][rows] storage), zeros outside the matrix, no divergent branches -- holds it across the
// K step's MFMAs and stores it to LDS afterwards.  A chunk is exactly one MFMA operand (row l % 32,
// k = 16 (l / 32) .. +15 of a 32-wide k-step).  Operands swapped in the MFMA as in the other kernels, so
// a lane holds four consecutive output columns and stores them with one 16-byte store.
#include "gemm_s8.h"

#include "gemm_gather8.h"

namespace gemm_impl {
namespace {

typedef int intx16 __attribute__((ext_vector_type(16)));

using namespace gather8;

template <int TW, int NSTAGE, int AMODE, int BMODE>
__global__ __launch_bounds__(256) void gemm_s8_kernel(GemmParams p) {
  constexpr bool a_kc = AMODE != MC, b_kc = BMODE != MC;
  constexpr int BM = 64 * TW, BN = 64 * TW;
  constexpr int OP_BYTES = BM * BKB;
  constexpr int STAGE = 2 * OP_BYTES;
  constexpr int NLD = OP_BYTES / (256 * 16);
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int tile_m = blockIdx.x / p.tiles_n, tile_n = blockIdx.x % p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int64_t bz = blockIdx.z;
  const int8_t* A = reinterpret_cast<const int8_t*>(p.a) + bz * p.sa;
  const int8_t* B = reinterpret_cast<const int8_t*>(p.b) + bz * p.sb;
  const int8_t* a_tile = a_kc ? A + (int64_t)m0 * p.lda : A + m0;
  const int8_t* b_tile = b_kc ? B + (int64_t)n0 * p.ldb : B + n0;
  const int64_t a_step = a_kc ? BKB : BKB * p.lda;
  const int64_t b_step = b_kc ? BKB : BKB * p.ldb;

  intx16 acc[TW][TW];
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < TW; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  const int KT = (p.K + BKB - 1) / BKB;
  auto load_step = [&](int kt, intx4 (&ga)[NLD], intx4 (&gb)[NLD]) {
    const int kleft = p.K - kt * BKB;  // <= 0 past the end: zeros
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      ga[i] = gather<AMODE>(a_tile, reinterpret_cast<const int8_t*>(p.a), p.lda, p.M - m0, kleft, i, tid);
      gb[i] = gather<BMODE>(b_tile, reinterpret_cast<const int8_t*>(p.b), p.ldb, p.N - n0, kleft, i, tid);
    }
    a_tile += a_step;
    b_tile += b_step;
  };
  auto store_step = [&](char* stage, const intx4 (&ga)[NLD], const intx4 (&gb)[NLD]) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      *reinterpret_cast<intx4*>(stage + i * 4096 + tid * 16) = ga[i];
      *reinterpret_cast<intx4*>(stage + OP_BYTES + i * 4096 + tid * 16) = gb[i];
    }
  };
  // Fragment of the 32-row slab t for k-step ks (32 k): lane l gets row l % 32, k = 32 ks + 16 (l / 32) .. +15.
  int fa_off[2], fb_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const int ra = wm * 32 * TW + l32, rb = wn * 32 * TW + l32;
    fa_off[ks] = ra * BKB + (((2 * ks + g) ^ swz4(ra)) << 4);
    fb_off[ks] = OP_BYTES + rb * BKB + (((2 * ks + g) ^ swz4(rb)) << 4);  // + 32 rows: same swizzle
  }

  {
    intx4 ga[NLD], gb[NLD];
    for (int st = 0; st < NSTAGE - 1; ++st) {
      load_step(st, ga, gb);
      store_step(lds + st * STAGE, ga, gb);
    }
  }
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + (kt % NSTAGE) * STAGE;
    char* wr = lds + ((kt + NSTAGE - 1) % NSTAGE) * STAGE;  // read during step kt - 1
    intx4 ga[NLD], gb[NLD];
    load_step(kt + NSTAGE - 1, ga, gb);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      intx4 fa[TW], fb[TW];
#pragma unroll
      for (int t = 0; t < TW; ++t) {
        fa[t] = *reinterpret_cast<const intx4*>(cur + fa_off[ks] + t * 32 * BKB);
        fb[t] = *reinterpret_cast<const intx4*>(cur + fb_off[ks] + t * 32 * BKB);
      }
#pragma unroll
      for (int ti = 0; ti < TW; ++ti)
#pragma unroll
        for (int tj = 0; tj < TW; ++tj)
          acc[ti][tj] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[tj], fa[ti], acc[ti][tj], 0, 0, 0);
    }
    store_step(wr, ga, gb);
    __syncthreads();  // step kt + NSTAGE - 1 is in LDS for every wave; every wave is done with `cur`
  }

  // acc[i][j][e] is out[m][n] with m = m0 + 32 TW wm + 32 i + lane % 32 and
  // n = n0 + 32 TW wn + 32 j + 8 (e / 4) + 4 (lane / 32) + e % 4.
  int32_t* out = reinterpret_cast<int32_t*>((p.out_alt[0] && bz > 0) ? p.out_alt[bz - 1] : p.out) + bz * p.sc;
#pragma unroll
  for (int i = 0; i < TW; ++i) {
    const int m = m0 + wm * 32 * TW + i * 32 + l32;
    if (m >= p.M) continue;
#pragma unroll
    for (int j = 0; j < TW; ++j)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd) {
        const int n = n0 + wn * 32 * TW + j * 32 + 8 * qd + 4 * g;
        if (n >= p.N) continue;
        const intx16 t = acc[i][j];
        const int64_t off = (int64_t)m * p.ldc + n;
        if (n + 4 <= p.N && off % 4 == 0) {
          *reinterpret_cast<intx4*>(out + off) = intx4{t[4 * qd], t[4 * qd + 1], t[4 * qd + 2], t[4 * qd + 3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < p.N) out[off + e] = t[4 * qd + e];
        }
      }
  }
}

template <int TW, int AMODE>
void launch_b(const GemmParams& p, int bmode, dim3 grid, hipStream_t st) {
  if (bmode == KC_VEC) hipLaunchKernelGGL((gemm_s8_kernel<TW, 4, AMODE, KC_VEC>), grid, dim3(256), 0, st, p);
  else if (bmode == KC_SCALAR) hipLaunchKernelGGL((gemm_s8_kernel<TW, 4, AMODE, KC_SCALAR>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((gemm_s8_kernel<TW, 4, AMODE, MC>), grid, dim3(256), 0, st, p);
}
template <int TW>
void launch_a(const GemmParams& p, int amode, int bmode, dim3 grid, hipStream_t st) {
  if (amode == KC_VEC) launch_b<TW, KC_VEC>(p, bmode, grid, st);
  else if (amode == KC_SCALAR) launch_b<TW, KC_SCALAR>(p, bmode, grid, st);
  else launch_b<TW, MC>(p, bmode, grid, st);
}

}  // namespace

void launch_gemm_s8(GemmParams& p, bool a_mc, bool b_mc, int batch, hipStream_t st) {
  const bool large = xmk::ceil_div(p.M, 128) * xmk::ceil_div(p.N, 128) * batch >= 256;
  const int edge = large ? 128 : 64;
  p.tiles_m = (int)xmk::ceil_div(p.M, edge);
  p.tiles_n = (int)xmk::ceil_div(p.N, edge);
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch);
  const int amode = a_mc ? MC : (p.vec_a >= 16 ? KC_VEC : KC_SCALAR);
  const int bmode = b_mc ? MC : (p.vec_b >= 16 ? KC_VEC : KC_SCALAR);
  if (large) launch_a<2>(p, amode, bmode, grid, st);
  else launch_a<1>(p, amode, bmode, grid, st);
}

}  // namespace gemm_impl
