/*
 * xmk_oracle.c — CPU restatement of the custom-call hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product path links, loads or
 * calls this file: it is the checker the parity tests, the smoke test and the
 * benchmark's cpu_baseline leg compare the HIP kernels against.
 *
 * Every function computes from the *rounded* inputs (bf16 / fp16 / e4m3fn bit
 * patterns), accumulates in double, applies the epilogue in the order the
 * reference applies it, and rounds once to the output type.
 *
 * What pins each function (tests/test_oracle_*.py):
 *   codecs            : exhaustive against torch's CPU bfloat16/float16/float8_e4m3fn
 *   xo_gemm           : numpy float64 matmul, identity, transpose identities, linearity in beta
 *   xo_fmha_fwd       : numpy brute force, V=1 => O=1, causal row 0 == V[0], LSE == logsumexp,
 *                       and the reference test's own closed form at its tolerance
 *                       (test/jax_ut.patch:978-998)
 *   xo_fmha_fwd_online: agrees with xo_fmha_fwd (restates fmha_forward.h:331-385)
 *   xo_int4_dequant   : numpy uint/float32 brute force + exhaustive 16 x {z,s} table.
 *                       PARITY UNPINNED against the reference: the reference snapshot has no
 *                       int4 kernel; the packing and rounding order are defined by include/xmk.h.
 *   xo_fp8_gemm       : numpy float64 over the decoded table.  PARITY UNPINNED against the
 *                       reference for the same reason (no fp8 GEMM in the snapshot).
 *   GEMM arithmetic   : the reference's inner loop lives in intel/xetla v0.3.7.2 and oneDNN v3.7
 *                       (xla/workspace.bzl:7-18,39-51), absent from the tree; the reference holds
 *                       no numeric GEMM vectors, so GEMM parity is pinned by mathematics only.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define XO_F16 10
#define XO_F32 11
#define XO_BF16 16
#define XO_F8E4M3FN 20

/* ------------------------------------------------------------------ codecs */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

uint16_t xo_f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u); /* quiet NaN */
  u += 0x7fffu + ((u >> 16) & 1u); /* round to nearest even */
  return (uint16_t)(u >> 16);
}
float xo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

uint16_t xo_f32_to_f16(float f) {
  uint32_t u = f32_bits(f);
  uint32_t sign = (u >> 16) & 0x8000u;
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  /* NaN */
  if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 rounds to inf */
  if (a < 0x33000001u) return (uint16_t)sign;              /* <= 2^-25 rounds to 0 */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7fffffu) | 0x800000u;
  uint32_t shift, half_bits;
  if (e < -14) { /* subnormal result: value = m * 2^(e-23); unit 2^-24 */
    shift = (uint32_t)(-e - 1);  /* 13 + (-14 - e) */
    half_bits = 0;
  } else {
    shift = 13;
    half_bits = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  if (rem > halfway || (rem == halfway && (q & 1u))) q++;
  return (uint16_t)(sign | (half_bits + q)); /* carry propagates into the exponent */
}
float xo_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
  if (e == 0x1f) return bits_f32(sign | 0x7f800000u | (m << 13));
  if (e == 0) {
    float v = (float)m * 5.9604644775390625e-08f; /* 2^-24 */
    return sign ? -v : v;
  }
  return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

/* OCP e4m3fn: bias 7, 3 mantissa bits, no infinity, S.1111.111 is NaN, max 448. */
float xo_e4m3fn_to_f32(uint8_t b) {
  uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
  float v;
  if (e == 0xf && m == 7) return bits_f32(0x7fc00000u | ((uint32_t)(b & 0x80u) << 24));
  if (e == 0) v = (float)m * 0.001953125f; /* 2^-9 */
  else v = ldexpf((float)(8u + m), (int)e - 10);
  return (b & 0x80u) ? -v : v;
}
/* Round to nearest even; anything that rounds above 448 becomes NaN (the
 * non-saturating conversion torch's CPU float8_e4m3fn cast performs). */
uint8_t xo_f32_to_e4m3fn(float f) {
  uint32_t u = f32_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
  float x = bits_f32(a);
  if (x >= 480.0f) return (uint8_t)(sign | 0x7fu); /* 464 is the 448/480 midpoint -> 448 (even) */
  if (x > 464.0f) return (uint8_t)(sign | 0x7fu);
  int e;
  (void)frexpf(x, &e); /* x = f * 2^e, f in [0.5,1) -> exponent of leading bit is e-1 */
  int lead = e - 1;
  if (x == 0.0f) return sign;
  int qexp = lead < -6 ? -9 : lead - 3; /* quantum = 2^qexp */
  double scaled = ldexp((double)x, -qexp);
  double r = nearbyint(scaled); /* default rounding mode: nearest even */
  float y = (float)ldexp(r, qexp);
  if (y > 448.0f) return (uint8_t)(sign | 0x7fu);
  if (y == 0.0f) return sign;
  int e2;
  (void)frexpf(y, &e2);
  int lead2 = e2 - 1;
  if (lead2 < -6) { /* subnormal */
    uint32_t m = (uint32_t)ldexpf(y, 9);
    return (uint8_t)(sign | m);
  }
  uint32_t m = (uint32_t)ldexpf(y, 3 - lead2) - 8u;
  return (uint8_t)(sign | ((uint32_t)(lead2 + 7) << 3) | m);
}

static inline float load_elem(const void* p, int dtype, int64_t i) {
  switch (dtype) {
    case XO_BF16: return xo_bf16_to_f32(((const uint16_t*)p)[i]);
    case XO_F16: return xo_f16_to_f32(((const uint16_t*)p)[i]);
    case XO_F8E4M3FN: return xo_e4m3fn_to_f32(((const uint8_t*)p)[i]);
    default: return ((const float*)p)[i];
  }
}
static inline void store_elem(void* p, int dtype, int64_t i, float v) {
  switch (dtype) {
    case XO_BF16: ((uint16_t*)p)[i] = xo_f32_to_bf16(v); break;
    case XO_F16: ((uint16_t*)p)[i] = xo_f32_to_f16(v); break;
    case XO_F8E4M3FN: ((uint8_t*)p)[i] = xo_f32_to_e4m3fn(v); break;
    default: ((float*)p)[i] = v; break;
  }
}

void xo_convert_from_f32(int dtype, const float* src, void* dst, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) store_elem(dst, dtype, i, src[i]);
}
void xo_convert_to_f32(int dtype, const void* src, float* dst, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) dst[i] = load_elem(src, dtype, i);
}

/* --------------------------------------------------- deterministic inputs */

/* Counter-based generator: element i of stream `seed` depends on (seed, i)
 * only, so any slice can be produced independently and in parallel. */
static inline uint64_t splitmix64(uint64_t x) {
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}
static inline uint64_t draw(uint64_t seed, uint64_t ctr) {
  return splitmix64(splitmix64(seed) ^ (ctr * 0xd1342543de82ef95ull + 0x632be59bd9b4e019ull));
}
static inline double unit_open(uint64_t r) { /* (0,1) */
  return ((double)(r >> 11) + 0.5) * (1.0 / 9007199254740992.0);
}

/* out[i] = scale * N(0,1), Box-Muller in double on counters 2i, 2i+1. */
void xo_fill_normal(float* out, int64_t n, uint64_t seed, float scale) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    double u1 = unit_open(draw(seed, 2ull * (uint64_t)i));
    double u2 = unit_open(draw(seed, 2ull * (uint64_t)i + 1ull));
    double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925 * u2);
    out[i] = (float)(z * (double)scale);
  }
}
void xo_fill_uniform(float* out, int64_t n, uint64_t seed, float lo, float hi) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    double u = unit_open(draw(seed, (uint64_t)i));
    out[i] = (float)((double)lo + u * ((double)hi - (double)lo));
  }
}
/* 32 random bits per word = 8 uniform nibbles. */
void xo_fill_words(uint32_t* out, int64_t n, uint64_t seed) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) out[i] = (uint32_t)(draw(seed, (uint64_t)i) >> 32);
}

/* -------------------------------------------------------------------- GEMM */

typedef struct xo_matrix {
  const void* data;
  int32_t transpose;
  int64_t num_rows, num_cols, batch_stride, leading_dim_stride;
} xo_matrix;

/* Epilogue numbering of SYCLGemm::GemmBackendEpilogue (onednn_matmul_utils.h:35-45). */
enum { EPI_DEFAULT, EPI_RELU, EPI_GELU, EPI_BIAS, EPI_BIAS_RELU, EPI_BIAS_GELU };

static inline float gelu_tanh(float x) {
  /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))): oneDNN eltwise_gelu_tanh
   * (onednn_matmul_utils.cc:447) and XeTLA gelu_fwd_op_t (hgemm_impl.h:331). */
  double xd = x;
  return (float)(0.5 * xd * (1.0 + tanh(0.7978845608028654 * (xd + 0.044715 * xd * xd * xd))));
}

/* Logical element (r, c) of an operand described like MatrixDescriptor
 * (matrix_descriptor.h:30-46; GetMatrixDesc onednn_matmul_utils.cc:206-218). */
static inline int64_t mat_index(const xo_matrix* m, int64_t b, int64_t r, int64_t c) {
  return b * m->batch_stride + (m->transpose ? c * m->leading_dim_stride + r
                                             : r * m->leading_dim_stride + c);
}

/*
 * out = act(alpha * lhs·rhs + beta * c + bias), the order of DoOnednnGemm
 * (onednn_matmul_utils.cc:439-448: append_sum(beta) before the eltwise) and
 * of the XeTLA chain BIAS -> RES_ADD(beta) (:273-289; epilogue_impl.h:75-85,
 * 153-163, 228-241).  A column-major output is handled as the reference does
 * in MakeBlasGemmCompatible (:513-530): element (r, c) of the logical product
 * lands at the transposed position.  out_f32 (optional) receives the
 * unrounded fp32 values in logical [batch, m, n] order.
 */
int xo_gemm(const xo_matrix* lhs, const xo_matrix* rhs, const xo_matrix* out, void* out_data,
            const void* c, const void* bias, int dtype_in, int dtype_out, int64_t batch,
            float alpha, float beta, int epilogue, float* out_f32) {
  int64_t m = lhs->transpose ? lhs->num_cols : lhs->num_rows;
  int64_t k = lhs->transpose ? lhs->num_rows : lhs->num_cols;
  int64_t k2 = rhs->transpose ? rhs->num_cols : rhs->num_rows;
  int64_t n = rhs->transpose ? rhs->num_rows : rhs->num_cols;
  if (k != k2) return 3;
  int has_bias = (epilogue == EPI_BIAS || epilogue == EPI_BIAS_RELU || epilogue == EPI_BIAS_GELU);
  if (epilogue < 0 || epilogue > EPI_BIAS_GELU) return 12;
  if (has_bias && !bias) return 3;
  /* c may alias out_data: read every addend before any store of this row. */
  for (int64_t b = 0; b < batch; ++b) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
      float* rowbuf = (float*)malloc(sizeof(float) * (size_t)n);
      for (int64_t j = 0; j < n; ++j) {
        double acc = 0.0;
        for (int64_t p = 0; p < k; ++p)
          acc += (double)load_elem(lhs->data, dtype_in, mat_index(lhs, b, i, p)) *
                 (double)load_elem(rhs->data, dtype_in, mat_index(rhs, b, p, j));
        float v = alpha * (float)acc;
        if (beta != 0.0f && c) v += beta * load_elem(c, dtype_out, mat_index(out, b, i, j));
        if (has_bias) v += load_elem(bias, dtype_in, j);
        if (epilogue == EPI_RELU || epilogue == EPI_BIAS_RELU) v = v > 0.0f ? v : 0.0f;
        if (epilogue == EPI_GELU || epilogue == EPI_BIAS_GELU) v = gelu_tanh(v);
        rowbuf[j] = v;
      }
      for (int64_t j = 0; j < n; ++j) {
        store_elem(out_data, dtype_out, mat_index(out, b, i, j), rowbuf[j]);
        if (out_f32) out_f32[(b * m + i) * n + j] = rowbuf[j];
      }
      free(rowbuf);
    }
  }
  return 0;
}

/* Fast path of the same arithmetic for packed row-major A[M,K], B[K,N] (or
 * B[N,K] when rhs_transpose), used for large parity shapes and as the timed
 * CPU baseline: operands decoded once to fp32, fp32 FMA accumulation in
 * blocks of 8 partial sums, double across blocks. */
int xo_gemm_packed(const void* a, const void* b, const void* bias, void* out, float* out_f32,
                   int dtype_in, int dtype_out, int64_t m, int64_t n, int64_t k,
                   int rhs_transpose, int epilogue, float scale) {
  float* af = (float*)malloc(sizeof(float) * (size_t)(m * k));
  float* bt = (float*)malloc(sizeof(float) * (size_t)(n * k)); /* [N,K] */
  if (!af || !bt) { free(af); free(bt); return 13; }
  xo_convert_to_f32(dtype_in, a, af, m * k);
  if (rhs_transpose) {
    xo_convert_to_f32(dtype_in, b, bt, n * k);
  } else {
#pragma omp parallel for schedule(static)
    for (int64_t j = 0; j < n; ++j)
      for (int64_t p = 0; p < k; ++p) bt[j * k + p] = load_elem(b, dtype_in, p * n + j);
  }
  int has_bias = (epilogue == EPI_BIAS || epilogue == EPI_BIAS_RELU || epilogue == EPI_BIAS_GELU);
#pragma omp parallel for schedule(dynamic, 4)
  for (int64_t i = 0; i < m; ++i) {
    const float* ar = af + i * k;
    for (int64_t j = 0; j < n; ++j) {
      const float* br = bt + j * k;
      double acc = 0.0;
      int64_t p = 0;
      for (; p + 256 <= k; p += 256) {
        float s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int64_t q = 0; q < 256; q += 8)
          for (int t = 0; t < 8; ++t) s[t] += ar[p + q + t] * br[p + q + t];
        acc += (double)((s[0] + s[1]) + (s[2] + s[3])) + (double)((s[4] + s[5]) + (s[6] + s[7]));
      }
      for (; p < k; ++p) acc += (double)ar[p] * (double)br[p];
      float v = scale * (float)acc;
      if (has_bias) v += load_elem(bias, dtype_in, j);
      if (epilogue == EPI_RELU || epilogue == EPI_BIAS_RELU) v = v > 0.0f ? v : 0.0f;
      if (epilogue == EPI_GELU || epilogue == EPI_BIAS_GELU) v = gelu_tanh(v);
      if (out) store_elem(out, dtype_out, i * n + j, v);
      if (out_f32) out_f32[i * n + j] = v;
    }
  }
  free(af);
  free(bt);
  return 0;
}

/* -------------------------------------------------------------------- int4 */

/* W[k,n] = f16_rne((f32(q) - f32(z)) * f32(s)); q = nibble (k % 8) of
 * qweight[k/8, n].  Separate fp32 subtract and multiply: the volatile
 * intermediate forbids contraction into an FMA. */
static inline uint16_t dequant_one(uint32_t word, int j, uint16_t s, uint16_t z) {
  float q = (float)((word >> (4 * j)) & 0xfu);
  volatile float d = q - xo_f16_to_f32(z);
  volatile float w = d * xo_f16_to_f32(s);
  return xo_f32_to_f16(w);
}
void xo_int4_dequant(const uint32_t* qweight, const uint16_t* scales, const uint16_t* zeros,
                     uint16_t* w_out, int64_t k, int64_t n, int64_t group) {
#pragma omp parallel for schedule(static)
  for (int64_t kk = 0; kk < k; ++kk) {
    int64_t g = kk / group;
    for (int64_t j = 0; j < n; ++j)
      w_out[kk * n + j] = dequant_one(qweight[(kk / 8) * n + j], (int)(kk % 8),
                                      scales[g * n + j], zeros[g * n + j]);
  }
}
/* out[m,n] = f16(sum_k f32(act[m,k]) * w[k,n] + f32(bias[n])), double accumulation, where
 * w[k,n] is the dequantised weight: the fp32 value (f32(q) - f32(z)) * f32(s) when
 * round_weights == 0 (the GEMM's contract: no intermediate rounding to fp16), or that value
 * rounded to fp16 (the output of xo_int4_dequant) when round_weights != 0. */
void xo_int4_gemm(const uint16_t* act, const uint32_t* qweight, const uint16_t* scales,
                  const uint16_t* zeros, const uint16_t* bias, uint16_t* out, float* out_f32,
                  int64_t m, int64_t k, int64_t n, int64_t group, int round_weights) {
  float* af = (float*)malloc(sizeof(float) * (size_t)(m * k));
  for (int64_t i = 0; i < m * k; ++i) af[i] = xo_f16_to_f32(act[i]);
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < n; ++j) {
    double* acc = (double*)calloc((size_t)m, sizeof(double));
    for (int64_t kk = 0; kk < k; ++kk) {
      int64_t g = kk / group;
      uint32_t word = qweight[(kk / 8) * n + j];
      float w;
      if (round_weights) {
        w = xo_f16_to_f32(dequant_one(word, (int)(kk % 8), scales[g * n + j], zeros[g * n + j]));
      } else {
        float q = (float)((word >> (4 * (kk % 8))) & 0xfu);
        volatile float d = q - xo_f16_to_f32(zeros[g * n + j]);
        volatile float wv = d * xo_f16_to_f32(scales[g * n + j]);
        w = wv;
      }
      for (int64_t i = 0; i < m; ++i) acc[i] += (double)af[i * k + kk] * (double)w;
    }
    for (int64_t i = 0; i < m; ++i) {
      float v = (float)acc[i];
      if (bias) v += xo_f16_to_f32(bias[j]);
      if (out) out[i * n + j] = xo_f32_to_f16(v);
      if (out_f32) out_f32[i * n + j] = v;
    }
    free(acc);
  }
  free(af);
}

/* --------------------------------------------------------------------- fp8 */

/* scale = amax / 448 (fp32); q = e4m3fn_rne(x / scale). */
void xo_fp8_quantize(const float* x, int64_t n, uint8_t* q, float* scale_out) {
  float amax = 0.0f;
  for (int64_t i = 0; i < n; ++i) {
    float a = fabsf(x[i]);
    if (a > amax) amax = a;
  }
  float scale = amax > 0.0f ? amax / 448.0f : 1.0f;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) q[i] = xo_f32_to_e4m3fn(x[i] / scale);
  *scale_out = scale;
}
/* out = bf16(a_scale * b_scale * sum f32(a) f32(b)). */
int xo_fp8_gemm(const uint8_t* a, const uint8_t* b, float a_scale, float b_scale, uint16_t* out,
                float* out_f32, int64_t m, int64_t n, int64_t k, int rhs_transpose) {
  return xo_gemm_packed(a, b, NULL, out, out_f32, XO_F8E4M3FN, XO_BF16, m, n, k, rhs_transpose,
                        EPI_DEFAULT, a_scale * b_scale);
}

/* --------------------------------------------------------------- attention */

/*
 * O = softmax(scale * Q K^T + bias + mask) V, two-pass in double, for
 * [first_unit, first_unit + num_units) of the B*N (batch, head) units.
 * Tensor layouts of RunFusedMHA (xetla_gpu_fused_mha_runner.cc:113-123):
 * Q [B,N,F,H], K [B,N,T,H], V [B,N,T,H], bias [B,N,F,T] (indexed by the unit
 * b*N+n, fmha_forward.h:235-241), out [B,N,F,H], lse fp32 [B*N,F] = m + log l
 * (fmha_forward.h:446).  Scores are scaled after the QK^T accumulate
 * (fmha_forward.h:266), bias added after scaling (:269-281).  Causal mask:
 * key x > query y is -inf, absolute indices, top-left aligned
 * (fmha_utils.h:45-96).  kv_unit_stride = elements between consecutive
 * units' K (and V) blocks (T*H when packed).
 */
void xo_fmha_fwd(int dtype, const void* q, const void* k, const void* v, const void* bias,
                 void* out, float* out_f32, float* lse, int64_t num_units, int64_t first_unit,
                 int64_t H, int64_t F, int64_t T, int64_t kv_unit_stride, float scale,
                 int causal, int64_t f_stride) {
  /* f_stride > 1: only query rows 0, f_stride, 2 f_stride, ... are computed (sampling). */
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
  for (int64_t u = first_unit; u < first_unit + num_units; ++u) {
    for (int64_t f = 0; f < F; ++f) {
      if (f % f_stride != 0) continue;
      double* s = (double*)malloc(sizeof(double) * (size_t)T);
      double* o = (double*)calloc((size_t)H, sizeof(double));
      float* qf = (float*)malloc(sizeof(float) * (size_t)H);
      for (int64_t h = 0; h < H; ++h) qf[h] = load_elem(q, dtype, (u * F + f) * H + h);
      int64_t tmax = causal ? (f + 1 < T ? f + 1 : T) : T;
      double mx = -INFINITY;
      for (int64_t t = 0; t < tmax; ++t) {
        double acc = 0.0;
        for (int64_t h = 0; h < H; ++h)
          acc += (double)qf[h] * (double)load_elem(k, dtype, u * kv_unit_stride + t * H + h);
        acc = (double)((float)acc * scale); /* fp32 S scaled by the fp32 scale */
        if (bias) acc += (double)load_elem(bias, dtype, (u * F + f) * T + t);
        s[t] = acc;
        if (acc > mx) mx = acc;
      }
      double l = 0.0;
      for (int64_t t = 0; t < tmax; ++t) {
        double p = exp(s[t] - mx);
        l += p;
        for (int64_t h = 0; h < H; ++h)
          o[h] += p * (double)load_elem(v, dtype, u * kv_unit_stride + t * H + h);
      }
      for (int64_t h = 0; h < H; ++h) {
        float val = (float)(o[h] / l);
        if (out) store_elem(out, dtype, (u * F + f) * H + h, val);
        if (out_f32) out_f32[(u * F + f) * H + h] = val;
      }
      if (lse) lse[u * F + f] = (float)(mx + log(l));
      free(s);
      free(o);
      free(qf);
    }
  }
}

/*
 * The reference's own recurrence (fmha_forward.h:331-385), key blocks of kBc:
 *   m' = max(m, rowmax S); l <- l e^{m-m'}; P = e^{S-m'}; l' = l + rowsum P;
 *   P <- P / l'; O <- O / (l'/l) + T(P) V    with P rounded to the element
 *   type before the second product (:378-384), fp32 state.
 * Exists to show that the closed form above and the reference's streaming
 * form agree to the tolerance the kernels are held to.
 */
void xo_fmha_fwd_online(int dtype, const void* q, const void* k, const void* v, const void* bias,
                        float* out_f32, int64_t num_units, int64_t H, int64_t F, int64_t T,
                        float scale, int causal, int64_t kBc) {
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
  for (int64_t u = 0; u < num_units; ++u) {
    for (int64_t f = 0; f < F; ++f) {
      float* o = (float*)calloc((size_t)H, sizeof(float));
      float* p = (float*)malloc(sizeof(float) * (size_t)kBc);
      float m = -INFINITY, l = 0.0f;
      for (int64_t t0 = 0; t0 < T; t0 += kBc) {
        if (causal && t0 > f) break; /* blocks past the diagonal are skipped (:544-546) */
        int64_t bc = T - t0 < kBc ? T - t0 : kBc;
        float bm = -INFINITY;
        for (int64_t t = 0; t < bc; ++t) {
          float acc = 0.0f;
          for (int64_t h = 0; h < H; ++h)
            acc += load_elem(q, dtype, (u * F + f) * H + h) *
                   load_elem(k, dtype, (u * T + t0 + t) * H + h);
          acc *= scale;
          if (bias) acc += load_elem(bias, dtype, (u * F + f) * T + t0 + t);
          if (causal && t0 + t > f) acc = -INFINITY;
          p[t] = acc;
          if (acc > bm) bm = acc;
        }
        float m_new = bm > m ? bm : m;
        l *= expf(m - m_new);
        float rs = 0.0f;
        for (int64_t t = 0; t < bc; ++t) { p[t] = expf(p[t] - m_new); rs += p[t]; }
        float l_new = l + rs;
        float o_scale = l_new / l; /* first block: l == 0 -> inf -> O/inf = 0 */
        for (int64_t h = 0; h < H; ++h) o[h] = o[h] / o_scale;
        for (int64_t t = 0; t < bc; ++t) {
          float pt = p[t] / l_new;
          uint16_t r = dtype == XO_BF16 ? xo_f32_to_bf16(pt) : xo_f32_to_f16(pt);
          pt = dtype == XO_BF16 ? xo_bf16_to_f32(r) : xo_f16_to_f32(r);
          for (int64_t h = 0; h < H; ++h)
            o[h] += pt * load_elem(v, dtype, (u * T + t0 + t) * H + h);
        }
        m = m_new;
        l = l_new;
      }
      for (int64_t h = 0; h < H; ++h) out_f32[(u * F + f) * H + h] = o[h];
      free(o);
      free(p);
    }
  }
}

/* Threads the OpenMP loops above will use (reported as cpu_baseline.cores). */
#ifdef _OPENMP
#include <omp.h>
int xo_num_threads(void) { return omp_get_max_threads(); }
#else
int xo_num_threads(void) { return 1; }
#endif
