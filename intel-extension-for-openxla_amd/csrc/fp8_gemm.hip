// FP8 (OCP e4m3fn) GEMM: out = bf16(d_scale * (a_scale * b_scale * A B + bias)), fp32 accumulation;
// d_scale and bias are optional.
//
// MFMA kernel: A [M,K] row-major and B stored [N,K] (both reduction-contiguous, the
// layout XLA's "__cublas$lt$matmul$f8" rewrite produces).  256x256 output tile per
// work-group (2x2 waves), K walked in steps of 64 bytes = one v_mfma_f32_32x32x64_f8f6f4
// k-step, in which a lane supplies 32 consecutive k of one row.  Operand tiles go from
// global memory straight into LDS (buffer_load ... lds) through the same 4-stage ring,
// swizzle and wait/barrier scheme as the 16-bit GEMM: a 64-byte fp8 row is byte for byte
// the 32-element 16-bit row that kernel's loader handles.  The per-tensor scales are read
// from device memory in the epilogue.
// B stored [K,N] (rhs_transpose == 0) takes the same kernel: its 64 k x BN tile goes into LDS as it
// lies in memory (n contiguous, the 16-bit GEMM's loader for that layout) and the fragments are read
// with ds_read_b64_tr_b8, which hands a lane 8 consecutive k of one column.
#include <utility>

#include "gemm_gather8.h"
#include "gemm_kernel.h"

namespace {

using gemm_impl::floatx16;
using gemm_impl::static_for;
using gemm_impl::u32x2;
using gemm_impl::u32x4;
using gemm_impl::zero16;
typedef int intx8 __attribute__((ext_vector_type(8)));

constexpr int BKB = 64;  // K step in bytes (= fp8 elements)
constexpr uint32_t kOob = gemm_impl::kOob;

struct Fp8Params {
  const uint8_t* a;
  const uint8_t* b;
  const float* a_scale;
  const float* b_scale;
  const float* d_scale;  // optional: multiplies the result after the bias
  const __bf16* bias;    // optional: [N], added to a_scale * b_scale * A B
  __bf16* out;
  int M, N, K;
  int tiles_m, tiles_n;
};

// out element = bf16(d_scale * (a_scale * b_scale * acc + bias[n])); `scale` = a_scale * b_scale.
struct Fp8Epilogue {
  float scale, post;
  const __bf16* bias;
  __device__ __forceinline__ explicit Fp8Epilogue(const Fp8Params& p)
      : scale(p.a_scale[0] * p.b_scale[0]), post(p.d_scale ? p.d_scale[0] : 1.0f), bias(p.bias) {}
  __device__ __forceinline__ bool plain() const { return !bias && post == 1.0f; }
  __device__ __forceinline__ __bf16 operator()(float acc, int n) const {
    float v = acc * scale;
    if (bias) v += (float)bias[n];
    return (__bf16)(v * post);
  }
};

// Per-lane LDS byte offsets of an operand's fragments: lane l of the 32-row slab t gets row
// 32 t + l%32, bytes 32 (l/32) .. +31 of the 64-byte row, i.e. the two 16-byte chunks 2 (l/32)
// and 2 (l/32) + 1, each XOR-swizzled like the loader placed them.  Adding 32 t rows does not
// change the swizzle.
struct Fp8Frag {
  int base[2];
  __device__ __forceinline__ void init(int row0, int lane) {
    const int row = row0 + (lane & 31);
    const int s = gemm_impl::swz<false, 0, 32>(row);
#pragma unroll
    for (int h = 0; h < 2; ++h) base[h] = row * BKB + ((((lane >> 5) * 2 + h) ^ s) << 4);
  }
  __device__ __forceinline__ intx8 read(const char* __restrict__ tile, int t) const {
    const u32x4 lo = *reinterpret_cast<const u32x4*>(tile + base[0] + t * 32 * BKB);
    const u32x4 hi = *reinterpret_cast<const u32x4*>(tile + base[1] + t * 32 * BKB);
    intx8 v;
    v[0] = (int)lo[0]; v[1] = (int)lo[1]; v[2] = (int)lo[2]; v[3] = (int)lo[3];
    v[4] = (int)hi[0]; v[5] = (int)hi[1]; v[6] = (int)hi[2]; v[7] = (int)hi[3];
    return v;
  }
};

// The same fragments from a tile stored [64 k][BN columns] (row = BN bytes, 16-byte chunks XOR-swizzled
// by the loader with swz<true, BN / 2, 64, 1>(k)).  ds_read_b64_tr_b8 works on blocks of 16 lanes: lane p
// of a block addresses row kb + p / 2, bytes cb + 8 (p % 2) .. +7 and receives column cb + p, rows
// kb .. kb + 7.  Blocks 0 and 1 of the wave cover columns 0..15 and 16..31 of the slab for k half 0,
// blocks 2 and 3 the same columns for k half 1; four reads, 8 rows apart, give a lane its 32 k.  The
// swizzle depends on k & 7 = p / 2 only, so one address per slab serves the four reads.
template <int BN, int T>
struct Fp8FragKN {
  int base[T];
  __device__ __forceinline__ void init(int col0, int lane) {
    const int p = lane & 15;
    const int k = (lane >> 5) * 32 + (p >> 1);
#pragma unroll
    for (int t = 0; t < T; ++t) {
      const int col = col0 + t * 32 + ((lane >> 4) & 1) * 16 + 8 * (p & 1);
      base[t] = k * BN + (((col >> 4) ^ gemm_impl::swz<true, BN / 2, 64, 1>(k)) << 4) + (col & 15);
    }
  }
  // t counts 32-column slabs from col0; only slabs this wave owns are read.
  __device__ __forceinline__ intx8 read(const char* __restrict__ tile, int t) const {
    typedef int int2v __attribute__((ext_vector_type(2)));
    typedef int2v __attribute__((address_space(3))) * lds_ptr;
    intx8 v;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int2v r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_ptr)(tile + base[t] + q * 8 * BN));
      v[2 * q] = r[0];
      v[2 * q + 1] = r[1];
    }
    return v;
  }
};

__device__ __forceinline__ floatx16 mfma_fp8(intx8 a, intx8 b, floatx16 c) {
  // cbsz = blgp = 0: both operands e4m3; block scales 127 = 2^0 (E8M0).
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 127, 0, 127);
}

template <int BM, int BN, int WGM, int WGN, int NSTAGE, bool BKN = false>
__global__ __launch_bounds__(WGM * WGN * 64) void fp8_gemm_kernel(Fp8Params p) {
  constexpr int NWAVES = WGM * WGN;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int A_BYTES = BM * BKB, B_BYTES = BN * BKB, STAGE = A_BYTES + B_BYTES;
  // The loader works in 2-byte units: BK = 32 units = 64 bytes.
  typedef gemm_impl::Loader<false, BM, 32, NWAVES> LoaderA;
  // B [n,k]: BN rows of 64 bytes; B [k,n]: 64 rows of BN bytes (BN / 2 two-byte units).
  typedef std::conditional_t<BKN, gemm_impl::Loader<true, BN / 2, 64, NWAVES, 1>, gemm_impl::Loader<false, BN, 32, NWAVES>>
      LoaderB;
  constexpr int LOADS = LoaderA::NL + LoaderB::NL;  // per wave per K step
  static_assert(NSTAGE >= 3, "the barrier leaves the running step's loads in flight");
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  int pid = blockIdx.x;
  const int ntiles = p.tiles_m * p.tiles_n;
  if (ntiles % 8 == 0) pid = (pid % 8) * (ntiles / 8) + pid / 8;  // one contiguous run of tiles per XCD
  constexpr int GM = 8;
  const int group = pid / (GM * p.tiles_n);
  const int first_m = group * GM;
  const int gsize = min(p.tiles_m - first_m, GM);
  const int tile_m = first_m + (pid % (GM * p.tiles_n)) % gsize;
  const int tile_n = (pid % (GM * p.tiles_n)) / gsize;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = zero16();

  LoaderA la;
  LoaderB lb;
  la.init(p.K / 2, p.M - m0, wave, lane);
  if constexpr (BKN) lb.init(p.N / 2, (p.N - n0) / 2, wave, lane);
  else lb.init(p.K / 2, p.N - n0, wave, lane);
  const uint8_t* a_tile = p.a + (int64_t)m0 * p.K;
  const uint8_t* b_tile = BKN ? p.b + n0 : p.b + (int64_t)n0 * p.K;
  const int64_t b_step = BKN ? (int64_t)BKB * p.N : BKB;  // bytes from one K step's B tile to the next
  // k of a K step that exist, in the unit the loader compares with: two-byte units along a
  // k-contiguous row, rows of the [k,n] tile.
  auto kleft_b = [&](int st) { return BKN ? p.K - st * BKB : (p.K - st * BKB) / 2; };
  const int KT = (p.K + BKB - 1) / BKB;

  // Prologue: K steps 0 .. NSTAGE-2.  Loads past the end of K write zeros, so every step issues
  // the same number of loads and the vmcnt arithmetic is uniform.
#pragma unroll
  for (int st = 0; st < NSTAGE - 1; ++st) {
    la.issue(a_tile, (p.K - st * BKB) / 2, lds + st * STAGE, wave);
    lb.issue(b_tile, kleft_b(st), lds + st * STAGE + A_BYTES, wave);
    a_tile += BKB;
    b_tile += b_step;
  }
  __builtin_amdgcn_s_waitcnt(gemm_impl::vmcnt_imm((NSTAGE - 2) * LOADS));  // step 0 has landed
  __builtin_amdgcn_s_barrier();

  Fp8Frag fa_addr;
  std::conditional_t<BKN, Fp8FragKN<BN, TN>, Fp8Frag> fb_addr;
  fa_addr.init(wm * WTM, lane);
  fb_addr.init(wn * WTN, lane);
  // Fragment registers: the B fragments of a step are double-buffered (those of step kt + 1 are
  // read while step kt computes); the A fragments rotate through two slots, A fragment i + 1
  // being read under the MFMAs of fragment i, and fragment 0 of the next step under the last.
  static_assert(TM % 2 == 0 && TN <= TM, "fragment rotation");
  intx8 fa[2], fb[2][TN];
  constexpr int NMFMA = TM * TN;
  // One K step kt: B fragments (buffer `par`) and A fragment 0 of step kt are in registers.  Once
  // step kt + 1 has landed for every wave (vmcnt + barrier; all reads issued so far are complete
  // too), issue the loads of step kt + NSTAGE - 1 into the stage step kt - 1 used, and run the
  // MFMAs of step kt while reading the rest of its A fragments from `cur` and the first fragments
  // of step kt + 1 from `nxt`.  The stages are distinct (__restrict__), so the compiler keeps the
  // loads in flight across the fragment reads.
  auto k_step = [&](auto PAR, const char* __restrict__ cur, const char* __restrict__ nxt, char* __restrict__ wr,
                    int kt) {
    constexpr int par = decltype(PAR)::value;
    const int kleft = (p.K - (kt + NSTAGE - 1) * BKB) / 2;
    const __amdgpu_buffer_rsrc_t ra = gemm_impl::make_rsrc(a_tile), rb = gemm_impl::make_rsrc(b_tile);
    __builtin_amdgcn_s_waitcnt(gemm_impl::vmcnt_imm((NSTAGE - 3) * LOADS) & ~(0xf << 8));  // and lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < LoaderA::NL; ++i) la.issue_one(i, ra, kleft, wr, wave);
#pragma unroll
    for (int i = 0; i < LoaderB::NL; ++i) lb.issue_one(i, rb, kleft_b(kt + NSTAGE - 1), wr + A_BYTES, wave);
    static_for<TM>([&](auto I) {
      constexpr int i = decltype(I)::value;
      if constexpr (i + 1 < TM) fa[(i + 1) & 1] = fa_addr.read(cur, i + 1);
      else fa[0] = fa_addr.read(nxt, 0);
      if constexpr (i < TN) fb[par ^ 1][i] = fb_addr.read(nxt + A_BYTES, i);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int jj = (i & 1) ? TN - 1 - j : j;  // boustrophedon: consecutive MFMAs share one operand
        acc[i][jj] = mfma_fp8(fb[par][jj], fa[i & 1], acc[i][jj]);
      }
    });
    // Issue order: each row of MFMAs starts with its LDS reads (4 x 16 bytes), the global loads
    // are spread evenly.
    static_for<NMFMA>([&](auto R) {
      constexpr int r = decltype(R)::value;
      if constexpr (r % TN == 0) __builtin_amdgcn_sched_group_barrier(0x100, (r / TN < TN) ? (BKN ? 6 : 4) : 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      if constexpr ((r + 1) * LOADS / NMFMA > r * LOADS / NMFMA) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    });
    __builtin_amdgcn_sched_barrier(0);
    a_tile += BKB;
    b_tile += b_step;
  };

#pragma unroll
  for (int j = 0; j < TN; ++j) fb[0][j] = fb_addr.read(lds + A_BYTES, j);
  fa[0] = fa_addr.read(lds, 0);
  for (int kt = 0; kt < KT; kt += 2) {
    k_step(std::integral_constant<int, 0>{}, lds + (kt % NSTAGE) * STAGE, lds + ((kt + 1) % NSTAGE) * STAGE,
           lds + ((kt + NSTAGE - 1) % NSTAGE) * STAGE, kt);
    if (kt + 1 < KT)
      k_step(std::integral_constant<int, 1>{}, lds + ((kt + 1) % NSTAGE) * STAGE,
             lds + ((kt + 2) % NSTAGE) * STAGE, lds + ((kt + NSTAGE) % NSTAGE) * STAGE, kt + 1);
  }
  __builtin_amdgcn_s_waitcnt(gemm_impl::vmcnt_imm(0));  // drain the zero-fill loads before LDS is released

  // acc[i][j][e] is out[m][n], m = m0 + wm WTM + 32 i + lane%32, n = n0 + wn WTN + 32 j + 8 (e/4) + 4 (lane/32) + e%4.
  const Fp8Epilogue epi(p);
  const float scale = epi.scale;
  static_assert(NSTAGE * STAGE >= BM * BN * 2, "the output tile is staged in the operand stages");
  // A bias or an output scale (both rare with a bf16 result) take the direct stores below.
  if (epi.plain() && m0 + BM <= p.M && n0 + BN <= p.N && p.N % 8 == 0 && reinterpret_cast<uintptr_t>(p.out) % 16 == 0) {
    // Tile fully inside (uniform over the work-group): round, lay out row-major in LDS and copy out
    // in whole row segments.
    gemm_impl::GemmParams q{};
    q.out = p.out;
    q.ldc = p.N;
    q.alpha = scale;
    q.act = gemm_impl::ACT_NONE;
    __builtin_amdgcn_s_barrier();  // every wave has read its last fragments
    gemm_impl::store_tile_via_lds<__bf16, false, WTM, WTN, TM, TN>(q, acc, lds + wave * (WTM * WTN * 2),
                                                                   m0 + wm * WTM, n0 + wn * WTN, 0, lane);
    return;
  }
  static_for<TM>([&](auto I) {
    constexpr int i = decltype(I)::value;
    const int m = m0 + wm * WTM + i * 32 + (lane & 31);
    static_for<TN>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const floatx16 t = acc[i][j];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * WTN + j * 32 + q * 8 + (lane >> 5) * 4;
        if (m < p.M && n < p.N) {  // N % 4 == 0: the four columns are all in range
          union { __bf16 e[4]; u32x2 w; } o;
          o.e[0] = epi(t[4 * q + 0], n);
          o.e[1] = epi(t[4 * q + 1], n + 1);
          o.e[2] = epi(t[4 * q + 2], n + 2);
          o.e[3] = epi(t[4 * q + 3], n + 3);
          *reinterpret_cast<u32x2*>(p.out + (int64_t)m * p.N + n) = o.w;
        }
      }
    });
  });
}

// Any layout, size and alignment on the matrix cores: the operands are gathered (gemm_gather8.h) into
// the k-contiguous LDS layout, 16-byte chunks of 16 k; a lane's two neighbouring chunks are one operand
// of v_mfma_scale_f32_32x32x64_f8f6f4 (row l % 32, k = 32 (l / 32) .. +31).  256 threads = 4 waves in
// 2 x 2, tile 64 TW x 64 TW x 64, 4 LDS stages; the structure of the int8 kernel (gemm_s8.hip).
template <int TW, int NSTAGE, int AMODE, int BMODE>
__global__ __launch_bounds__(256) void fp8_gemm_gather_kernel(Fp8Params p) {
  using namespace gather8;
  constexpr bool b_kc = BMODE != MC;
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
  const int8_t* A = reinterpret_cast<const int8_t*>(p.a);
  const int8_t* B = reinterpret_cast<const int8_t*>(p.b);
  const int8_t* a_tile = A + (int64_t)m0 * p.K;                       // A is [M, K]
  const int8_t* b_tile = b_kc ? B + (int64_t)n0 * p.K : B + n0;       // B is [N, K] or [K, N]
  const int64_t ldb = b_kc ? p.K : p.N;
  const int64_t b_step = b_kc ? BKB : (int64_t)BKB * p.N;

  floatx16 acc[TW][TW];
#pragma unroll
  for (int i = 0; i < TW; ++i)
#pragma unroll
    for (int j = 0; j < TW; ++j) acc[i][j] = zero16();

  const int KT = (p.K + BKB - 1) / BKB;
  auto load_step = [&](int kt, intx4 (&ga)[NLD], intx4 (&gb)[NLD]) {
    const int kleft = p.K - kt * BKB;  // <= 0 past the end: zeros (fp8 zero is the zero byte)
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      ga[i] = gather<AMODE>(a_tile, A, p.K, p.M - m0, kleft, i, tid);
      gb[i] = gather<BMODE>(b_tile, B, ldb, p.N - n0, kleft, i, tid);
    }
    a_tile += BKB;
    b_tile += b_step;
  };
  auto store_step = [&](char* stage, const intx4 (&ga)[NLD], const intx4 (&gb)[NLD]) {
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      *reinterpret_cast<intx4*>(stage + i * 4096 + tid * 16) = ga[i];
      *reinterpret_cast<intx4*>(stage + OP_BYTES + i * 4096 + tid * 16) = gb[i];
    }
  };
  Fp8Frag fa_addr, fb_addr;
  fa_addr.init(wm * 32 * TW, lane);
  fb_addr.init(wn * 32 * TW, lane);

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
    intx8 fa[TW], fb[TW];
#pragma unroll
    for (int t = 0; t < TW; ++t) {
      fa[t] = fa_addr.read(cur, t);
      fb[t] = fb_addr.read(cur + OP_BYTES, t);
    }
#pragma unroll
    for (int ti = 0; ti < TW; ++ti)
#pragma unroll
      for (int tj = 0; tj < TW; ++tj) acc[ti][tj] = mfma_fp8(fb[tj], fa[ti], acc[ti][tj]);
    store_step(wr, ga, gb);
    __syncthreads();  // step kt + NSTAGE - 1 is in LDS for every wave; every wave is done with `cur`
  }

  // acc[i][j][e] is out[m][n], m = m0 + 32 TW wm + 32 i + lane % 32, n = n0 + 32 TW wn + 32 j + 8 (e/4) + 4 (lane/32) + e%4.
  const Fp8Epilogue epi(p);
  gemm_impl::GemmParams q{};
  q.out = p.out;
  q.M = p.M;
  q.N = p.N;
  q.ldc = p.N;
  q.alpha = epi.scale;
  q.act = gemm_impl::ACT_NONE;
#pragma unroll
  for (int i = 0; i < TW; ++i) {
    const int m = m0 + wm * 32 * TW + i * 32 + l32;
#pragma unroll
    for (int j = 0; j < TW; ++j) {
      const floatx16 t = acc[i][j];
      const int nb = n0 + wn * 32 * TW + j * 32 + g * 4;
      if (epi.plain()) {
        gemm_impl::store_quad<__bf16, false>(q, gemm_impl::floatx4{t[0], t[1], t[2], t[3]}, m, nb, 0);
        gemm_impl::store_quad<__bf16, false>(q, gemm_impl::floatx4{t[4], t[5], t[6], t[7]}, m, nb + 8, 0);
        gemm_impl::store_quad<__bf16, false>(q, gemm_impl::floatx4{t[8], t[9], t[10], t[11]}, m, nb + 16, 0);
        gemm_impl::store_quad<__bf16, false>(q, gemm_impl::floatx4{t[12], t[13], t[14], t[15]}, m, nb + 24, 0);
      } else if (m < p.M) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int n = nb + 8 * (e / 4) + e % 4;
          if (n < p.N) p.out[(int64_t)m * p.N + n] = epi(t[e], n);
        }
      }
    }
  }
}

template <int TW, int AMODE>
void launch_gather_b(const Fp8Params& p, int bmode, dim3 grid, hipStream_t st) {
  using namespace gather8;
  if (bmode == KC_VEC) hipLaunchKernelGGL((fp8_gemm_gather_kernel<TW, 4, AMODE, KC_VEC>), grid, dim3(256), 0, st, p);
  else if (bmode == KC_SCALAR) hipLaunchKernelGGL((fp8_gemm_gather_kernel<TW, 4, AMODE, KC_SCALAR>), grid, dim3(256), 0, st, p);
  else hipLaunchKernelGGL((fp8_gemm_gather_kernel<TW, 4, AMODE, MC>), grid, dim3(256), 0, st, p);
}

// a_vec / b_vec: 16-byte aligned pointer and K % 16 == 0 (the k-contiguous operand can be read 16 bytes at a time).
void launch_gather(Fp8Params& p, bool rhs_is_nk, bool a_vec, bool b_vec, hipStream_t st) {
  using namespace gather8;
  const bool large = xmk::ceil_div(p.M, 128) * xmk::ceil_div(p.N, 128) >= 256;
  const int edge = large ? 128 : 64;
  p.tiles_m = (int)xmk::ceil_div(p.M, edge);
  p.tiles_n = (int)xmk::ceil_div(p.N, edge);
  const dim3 grid((unsigned)(p.tiles_m * p.tiles_n));
  const int bmode = !rhs_is_nk ? MC : (b_vec ? KC_VEC : KC_SCALAR);
  if (large) {
    if (a_vec) launch_gather_b<2, KC_VEC>(p, bmode, grid, st);
    else launch_gather_b<2, KC_SCALAR>(p, bmode, grid, st);
  } else {
    if (a_vec) launch_gather_b<1, KC_VEC>(p, bmode, grid, st);
    else launch_gather_b<1, KC_SCALAR>(p, bmode, grid, st);
  }
}

// Plain tiled kernel for outputs that are not 8-byte aligned: 64x64 tile, fp8 decoded with the hardware
// conversion while staging, fp32 FMA.
__global__ __launch_bounds__(256) void fp8_gemm_generic_kernel(Fp8Params p, int rhs_transpose) {
  __shared__ float As[16][65];
  __shared__ float Bs[16][65];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < p.K; k0 += 16) {
    for (int e = threadIdx.x; e < 16 * 64; e += 256) {
      const int kk = e / 64, r = e % 64, k = k0 + kk;
      float av = 0.f, bv = 0.f;
      if (k < p.K && m0 + r < p.M)
        av = __builtin_amdgcn_cvt_f32_fp8((int)p.a[(int64_t)(m0 + r) * p.K + k], 0);
      if (k < p.K && n0 + r < p.N) {
        const int64_t i = rhs_transpose ? (int64_t)(n0 + r) * p.K + k : (int64_t)k * p.N + (n0 + r);
        bv = __builtin_amdgcn_cvt_f32_fp8((int)p.b[i], 0);
      }
      As[kk][r] = av;
      Bs[kk][r] = bv;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; b[i] = Bs[kk][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  const Fp8Epilogue epi(p);
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < p.M && n < p.N) p.out[(int64_t)m * p.N + n] = epi(acc[i][j], n);
    }
}

}  // namespace

extern "C" int xmk_fp8_gemm(const void* a, const void* b, const float* a_scale, const float* b_scale,
                            void* out, int64_t m, int64_t n, int64_t k, int32_t rhs_transpose,
                            void* stream) {
  return xmk_fp8_gemm_ex(a, b, a_scale, b_scale, nullptr, nullptr, out, m, n, k, rhs_transpose, stream);
}

extern "C" int xmk_fp8_gemm_ex(const void* a, const void* b, const float* a_scale, const float* b_scale,
                               const float* d_scale, const void* bias, void* out, int64_t m, int64_t n, int64_t k,
                               int32_t rhs_transpose, void* stream) {
  if (!a || !b || !a_scale || !b_scale || !out) return xmk::fail(XMK_INVALID_ARGUMENT, "fp8_gemm: null pointer");
  if (m <= 0 || n <= 0 || k <= 0) return xmk::fail(XMK_INVALID_ARGUMENT, "fp8_gemm: empty dimension");
  if (m > (1 << 30) || n > (1 << 30) || k > (1 << 30))
    return xmk::fail(XMK_INVALID_ARGUMENT, "fp8_gemm: dimension too large");
  Fp8Params p;
  p.a = (const uint8_t*)a; p.b = (const uint8_t*)b; p.a_scale = a_scale; p.b_scale = b_scale;
  p.d_scale = d_scale; p.bias = (const __bf16*)bias;
  p.out = (__bf16*)out; p.M = (int)m; p.N = (int)n; p.K = (int)k;
  hipStream_t st = (hipStream_t)stream;
  // The direct-to-LDS kernel: A rows and the stored rows of B start on 16-byte boundaries and hold whole
  // 16-byte chunks; one K step's tile of either operand lies within the 2 GiB a buffer descriptor spans.
  const bool fast_nk = rhs_transpose != 0 && k % 16 == 0 && n % 4 == 0 && 256 * k < (int64_t)kOob;
  const bool fast_kn = rhs_transpose == 0 && k % 16 == 0 && n % 16 == 0 && 256 * k < (int64_t)kOob &&
                       64 * n < (int64_t)kOob;
  if ((fast_nk || fast_kn) && xmk::aligned(a, 16) && xmk::aligned(b, 16) && xmk::aligned(out, 8)) {
    const bool big = xmk::ceil_div(m, 256) * xmk::ceil_div(n, 256) >= 256;
    // Between the two: about one 256 x 128 tile per CU (the 16-bit GEMM's third tile, for the same shapes).
    static const char* tile_env = getenv("XMK_FP8_TILE");
    const int64_t mid_tiles = xmk::ceil_div(m, 256) * xmk::ceil_div(n, 128);
    const bool mid = tile_env ? atoi(tile_env) == 1 : (!big && mid_tiles >= 192 && mid_tiles <= 256);
    xmk::trace("fp8_gemm m=%lld n=%lld k=%lld rhs_t=%d -> %s", (long long)m, (long long)n, (long long)k, rhs_transpose,
               mid ? "mfma_256x128" : big ? "mfma_256x256" : "mfma_128x128");
    if (mid) {
      p.tiles_m = (int)xmk::ceil_div(m, 256); p.tiles_n = (int)xmk::ceil_div(n, 128);
      if (fast_kn) hipLaunchKernelGGL((fp8_gemm_kernel<256, 128, 2, 2, 4, true>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, st, p);
      else hipLaunchKernelGGL((fp8_gemm_kernel<256, 128, 2, 2, 4>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, st, p);
    } else if (tile_env ? atoi(tile_env) == 2 : big) {
      p.tiles_m = (int)xmk::ceil_div(m, 256); p.tiles_n = (int)xmk::ceil_div(n, 256);
      if (fast_kn) hipLaunchKernelGGL((fp8_gemm_kernel<256, 256, 2, 4, 4, true>), dim3(p.tiles_m * p.tiles_n), dim3(512), 0, st, p);
      else hipLaunchKernelGGL((fp8_gemm_kernel<256, 256, 2, 4, 4>), dim3(p.tiles_m * p.tiles_n), dim3(512), 0, st, p);
    } else {
      p.tiles_m = (int)xmk::ceil_div(m, 128); p.tiles_n = (int)xmk::ceil_div(n, 128);
      if (fast_kn) hipLaunchKernelGGL((fp8_gemm_kernel<128, 128, 2, 2, 4, true>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, st, p);
      else hipLaunchKernelGGL((fp8_gemm_kernel<128, 128, 2, 2, 4>), dim3(p.tiles_m * p.tiles_n), dim3(256), 0, st, p);
    }
  } else if (xmk::aligned(out, 8) && (int64_t)m * k < (int64_t)1 << 40) {
    xmk::trace("fp8_gemm m=%lld n=%lld k=%lld rhs_t=%d -> mfma_gather", (long long)m, (long long)n, (long long)k,
               rhs_transpose);
    launch_gather(p, rhs_transpose != 0, k % 16 == 0 && xmk::aligned(a, 16), k % 16 == 0 && xmk::aligned(b, 16), st);
  } else {
    xmk::trace("fp8_gemm m=%lld n=%lld k=%lld rhs_t=%d -> generic_64x64", (long long)m, (long long)n,
               (long long)k, rhs_transpose);
    hipLaunchKernelGGL(fp8_gemm_generic_kernel, dim3((unsigned)xmk::ceil_div(n, 64), (unsigned)xmk::ceil_div(m, 64)),
                       dim3(256), 0, st, p, (int)rhs_transpose);
  }
  return xmk::check_launch("fp8_gemm");
}
