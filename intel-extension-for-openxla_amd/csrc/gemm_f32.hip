// fp32 x fp32 -> fp32 GEMM on the matrix cores (v_mfma_f32_32x32x2_f32), any layout and alignment.
// The reference runs these products through oneDNN (onednn_matmul_utils.cc:394-491, dtype triple
// :605-610).
//
// Work-group 256 threads = 4 waves in 2 x 2, tile 128 x 128 x 16 (64 x 64 x 16 for small products),
// 4 LDS stages.  Both operands are laid out k-contiguous in LDS ([row][16 floats], 64-byte rows, XOR-swizzled 16-byte chunks) whatever
// their layout in memory: every lane gathers one 16-byte chunk (four consecutive k of one row or
// column) per operand half -- one vector load where the operand is k-contiguous and aligned, four
// scalar loads otherwise, zeros outside the matrix, no divergent branches -- keeps it in registers across the K step's MFMAs
// and stores it to LDS afterwards.  fp32 MFMAs are slow enough (64 flop per cycle per SIMD) that the
// loads never limit the kernel; two work-groups per CU cover their latency.
// A lane's chunk of four k feeds four MFMAs (k = j and 4 + j of an 8-wide k-step for the two lane
// halves), the same permutation for both operands.  As in the 16-bit kernel the operands are swapped in
// the MFMA so that a lane holds four consecutive output columns, and the epilogue is shared with it.
#include "gemm_f32.h"

namespace gemm_impl {

template <> struct Elem<float> {
  static __device__ __forceinline__ float to_f32(float v) { return v; }
  static __device__ __forceinline__ uint16_t from_f32(float) { return 0; }  // fp32 outputs only
};

namespace {

constexpr int BKF = 16;
constexpr int ROWB = BKF * 4;           // bytes of one LDS row

__device__ __forceinline__ int swz4(int row) { return (row >> 2) & 3; }

// How an operand is fetched: k-contiguous with one aligned 16-byte load per chunk, k-contiguous element by
// element, or from [K][rows] storage (four rows of k apart).
enum : int { KC_VEC = 0, KC_SCALAR = 1, MC = 2 };

// Chunk i of this thread for one operand: LDS bytes [i * 4096 + tid * 16, +16) = row i * 64 + tid / 4,
// position tid % 4, which holds logical chunk (tid % 4) ^ swz4(row) = k 4 c .. 4 c + 3 of the K step.
// Branch-free: lanes outside the matrix load from `safe` (the operand's first element) and select zero,
// so that all loads of a K step are issued back to back and waited for once, after the MFMAs.
template <int MODE>
__device__ __forceinline__ floatx4 gather(const float* base, const float* safe, int64_t ld, int valid, int kleft,
                                          int i, int tid) {
  const int row = i * 64 + (tid >> 2);
  const int k = ((tid & 3) ^ swz4(row)) * 4;
  const bool in = row < valid;
  floatx4 v;
  if constexpr (MODE == KC_VEC) {  // K % 4 == 0: the chunk is inside the row or outside as a whole
    const bool ok = in && k < kleft;
    v = *reinterpret_cast<const floatx4*>(ok ? base + (int64_t)row * ld + k : safe);
    if (!ok) v = floatx4{0.f, 0.f, 0.f, 0.f};
  } else {
    const float* src = MODE == KC_SCALAR ? base + (int64_t)row * ld + k : base + (int64_t)k * ld + row;
    const int64_t step = MODE == KC_SCALAR ? 1 : ld;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = in && k + j < kleft;
      const float x = *(ok ? src + j * step : safe);
      v[j] = ok ? x : 0.f;
    }
  }
  return v;
}

// TW: 32-row slabs per wave in each direction; the tile is 64 TW x 64 TW (128 x 128 for large products,
// 64 x 64 where that leaves CUs idle).  NSTAGE: LDS stages; 4 of the large tile are 64 KB, which also keeps
// the work-groups per CU at two, so that e.g. 1024 tiles fill 512 slots twice instead of 768 slots 1.3 times.
template <int TW, int NSTAGE, int AMODE, int BMODE>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmParams p) {
  constexpr bool a_kc = AMODE != MC, b_kc = BMODE != MC;
  constexpr int BM = 64 * TW, BN = 64 * TW;
  constexpr int OP_BYTES = BM * ROWB;         // one operand tile
  constexpr int STAGE = 2 * OP_BYTES;
  constexpr int NLD = OP_BYTES / (256 * 16);  // 16-byte chunks per lane per operand and K step
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, g = lane >> 5;
  const int tile_m = blockIdx.x / p.tiles_n, tile_n = blockIdx.x % p.tiles_n;
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int64_t bz = blockIdx.z;
  const float* A = reinterpret_cast<const float*>(p.a) + bz * p.sa;
  const float* B = reinterpret_cast<const float*>(p.b) + bz * p.sb;
  // Tile origins; one K step further is +BKF elements (k-contiguous) or +BKF rows.
  const float* a_tile = a_kc ? A + (int64_t)m0 * p.lda : A + m0;
  const float* b_tile = b_kc ? B + (int64_t)n0 * p.ldb : B + n0;
  const int64_t a_step = a_kc ? BKF : BKF * p.lda;
  const int64_t b_step = b_kc ? BKF : BKF * p.ldb;

  floatx16 acc[TW][TW];
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < TW; ++j) acc[i][j] = zero16();

  const int KT = (p.K + BKF - 1) / BKF;
  auto load_step = [&](int kt, floatx4 (&ga)[NLD], floatx4 (&gb)[NLD]) {
    const int kleft = p.K - kt * BKF;  // <= 0 past the end: zeros
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      ga[i] = gather<AMODE>(a_tile, reinterpret_cast<const float*>(p.a), p.lda, p.M - m0, kleft, i, tid);
      gb[i] = gather<BMODE>(b_tile, reinterpret_cast<const float*>(p.b), p.ldb, p.N - n0, kleft, i, tid);
    }
    a_tile += a_step;
    b_tile += b_step;
  };
  auto store_step = [&](char* stage, const floatx4 (&ga)[NLD], const floatx4 (&gb)[NLD]) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      *reinterpret_cast<floatx4*>(stage + i * 4096 + tid * 16) = ga[i];
      *reinterpret_cast<floatx4*>(stage + OP_BYTES + i * 4096 + tid * 16) = gb[i];
    }
  };
  // Fragment of the 32-row slab t for k-step ks (8 k): lane l gets row l % 32, k = 8 ks + 4 (l / 32) .. +3.
  int fa_off[2], fb_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    const int ra = wm * 32 * TW + l32, rb = wn * 32 * TW + l32;
    fa_off[ks] = ra * ROWB + (((2 * ks + g) ^ swz4(ra)) << 4);
    fb_off[ks] = OP_BYTES + rb * ROWB + (((2 * ks + g) ^ swz4(rb)) << 4);  // + 32 rows: same swizzle
  }

  // Prologue: K steps 0 .. NSTAGE - 2 go to stages 0 .. NSTAGE - 2.
  {
    floatx4 ga[NLD], gb[NLD];
    for (int st = 0; st < NSTAGE - 1; ++st) {
      load_step(st, ga, gb);
      store_step(lds + st * STAGE, ga, gb);
    }
  }
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + (kt % NSTAGE) * STAGE;
    char* wr = lds + ((kt + NSTAGE - 1) % NSTAGE) * STAGE;  // read during step kt - 1
    floatx4 ga[NLD], gb[NLD];
    load_step(kt + NSTAGE - 1, ga, gb);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      floatx4 fa[TW], fb[TW];
#pragma unroll
      for (int t = 0; t < TW; ++t) {
        fa[t] = *reinterpret_cast<const floatx4*>(cur + fa_off[ks] + t * 32 * ROWB);
        fb[t] = *reinterpret_cast<const floatx4*>(cur + fb_off[ks] + t * 32 * ROWB);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int ti = 0; ti < TW; ++ti)
#pragma unroll
          for (int tj = 0; tj < TW; ++tj)
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[tj][j], fa[ti][j], acc[ti][tj], 0, 0, 0);
    }
    store_step(wr, ga, gb);
    __syncthreads();  // step kt + NSTAGE - 1 is in LDS for every wave; every wave is done with `cur`
  }

  // Epilogue: acc[i][j][e] is out[m][n] with m = m0 + 32 TW wm + 32 i + lane % 32 and
  // n = n0 + 32 TW wn + 32 j + 8 (e / 4) + 4 (lane / 32) + e % 4.
  const int64_t coff = bz * p.sc;
  GemmParams q = p;
  if (p.out_alt[0] && bz > 0) q.out = p.out_alt[bz - 1];
  if (p.bias) q.bias = reinterpret_cast<const float*>(p.bias) + bz * p.sbias;
#pragma unroll
  for (int i = 0; i < TW; ++i) {
    const int m = m0 + wm * 32 * TW + i * 32 + l32;
#pragma unroll
    for (int j = 0; j < TW; ++j) {
      const floatx16 t = acc[i][j];
      const int nb = n0 + wn * 32 * TW + j * 32 + g * 4;
      store_quad<float, true>(q, floatx4{t[0], t[1], t[2], t[3]}, m, nb, coff);
      store_quad<float, true>(q, floatx4{t[4], t[5], t[6], t[7]}, m, nb + 8, coff);
      store_quad<float, true>(q, floatx4{t[8], t[9], t[10], t[11]}, m, nb + 16, coff);
      store_quad<float, true>(q, floatx4{t[12], t[13], t[14], t[15]}, m, nb + 24, coff);
    }
  }
}

}  // namespace

namespace {
template <int TW, int AMODE>
void launch_b(const GemmParams& p, int bmode, dim3 grid, hipStream_t st) {
  if (bmode == KC_VEC) hipLaunchKernelGGL((gemm_f32_kernel<TW, 4, AMODE, KC_VEC>), grid, dim3(256), 0, st, p);
  else if (bmode == KC_SCALAR) hipLaunchKernelGGL((gemm_f32_kernel<TW, 4, AMODE, KC_SCALAR>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((gemm_f32_kernel<TW, 4, AMODE, MC>), grid, dim3(256), 0, st, p);
}
template <int TW>
void launch_a(const GemmParams& p, int amode, int bmode, dim3 grid, hipStream_t st) {
  if (amode == KC_VEC) launch_b<TW, KC_VEC>(p, bmode, grid, st);
  else if (amode == KC_SCALAR) launch_b<TW, KC_SCALAR>(p, bmode, grid, st);
  else launch_b<TW, MC>(p, bmode, grid, st);
}
}  // namespace

void launch_gemm_f32(GemmParams& p, bool a_mc, bool b_mc, int batch, hipStream_t st) {
  // 128 x 128 tiles when they give every CU work, else 64 x 64.
  const bool large = xmk::ceil_div(p.M, 128) * xmk::ceil_div(p.N, 128) * batch >= 256;
  const int edge = large ? 128 : 64;
  p.tiles_m = (int)xmk::ceil_div(p.M, edge);
  p.tiles_n = (int)xmk::ceil_div(p.N, edge);
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n), 1, (unsigned)batch);
  const int amode = a_mc ? MC : (p.vec_a >= 4 ? KC_VEC : KC_SCALAR);
  const int bmode = b_mc ? MC : (p.vec_b >= 4 ? KC_VEC : KC_SCALAR);
  if (large) launch_a<2>(p, amode, bmode, grid, st);
  else launch_a<1>(p, amode, bmode, grid, st);
}

}  // namespace gemm_impl
