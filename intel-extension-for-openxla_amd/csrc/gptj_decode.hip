// GPT-J-shaped decode step on int4 weights: the LayerNorm kernel and the host loop that strings it
// together with the int4 GEMM (whose q/k/v epilogue applies the rotary embedding and appends to the
// KV cache) and the split-key decode attention.  Everything is enqueued on one stream, in
// order, with no host synchronisation, so a caller can capture the whole step in a HIP graph.
#include "common.h"
#include "int4_gemm.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// y = (x - mean) / sqrt(var + eps) * gamma + beta, one work-group per row, fp32 statistics.
// A thread keeps its elements (8 per 16-byte load, up to LN_MAXV loads) in registers between the
// statistics and the normalisation, so the row is read once.  d % 8 == 0, d <= 512 * 8 * LN_MAXV.
// With x_out != NULL the row is first assembled from the previous block's pieces,
//     x = fp16( x_in + sum_s p1[s] + sum_s p2[s] + bias2 )
// (p1, p2: fp32 partial sums [ks][32][d] of the K-split out_proj and fc_out GEMMs, added in slice
// order), written to x_out, and normalised from the rounded value.
constexpr int LN_NT = 512, LN_MAXV = 4;
typedef uint32_t ln_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(LN_NT) void layernorm_kernel(const _Float16* __restrict__ x,
                                                          const _Float16* __restrict__ gamma,
                                                          const _Float16* __restrict__ beta,
                                                          _Float16* __restrict__ y, int d, float eps,
                                                          const float* __restrict__ p1, int ks1,
                                                          const float* __restrict__ p2, int ks2,
                                                          const _Float16* __restrict__ bias2,
                                                          _Float16* __restrict__ x_out) {
  typedef float ln_f32x4 __attribute__((ext_vector_type(4)));
  __shared__ float s_part[2][LN_NT / 64];
  union Pack { ln_u32x4 u; _Float16 e[8]; };
  const _Float16* xr = x + (size_t)blockIdx.x * d;
  Pack v[LN_MAXV];
  // gamma and beta do not depend on the statistics: fetched up front, their latency passes under the row's
  // (a load cannot move up across the barrier below by itself)
  Pack gm[LN_MAXV], bt[LN_MAXV];
#pragma unroll
  for (int j = 0; j < LN_MAXV; ++j) {
    const int i = (threadIdx.x + j * LN_NT) * 8;
    if (i < d) {
      gm[j].u = *reinterpret_cast<const ln_u32x4*>(gamma + i);
      bt[j].u = *reinterpret_cast<const ln_u32x4*>(beta + i);
    }
  }
  float s = 0.f, ss = 0.f;
#pragma unroll
  for (int j = 0; j < LN_MAXV; ++j) {
    const int i = (threadIdx.x + j * LN_NT) * 8;
    if (i < d) {
      v[j].u = *reinterpret_cast<const ln_u32x4*>(xr + i);
      if (x_out) {
        float f[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = (float)v[j].e[e];
        // All slices are loaded before the first is added: with four work-groups in the whole launch
        // the chain of load latencies is what this kernel costs.  Added in slice order.
        auto add_slices = [&](const float* p, int ks) {
          ln_f32x4 lo[xmk::kInt4MaxSplit], hi[xmk::kInt4MaxSplit];
#pragma unroll
          for (int sl = 0; sl < xmk::kInt4MaxSplit; ++sl)
            if (sl < ks) {
              const float* q = p + ((size_t)sl * 32 + blockIdx.x) * d + i;
              lo[sl] = *reinterpret_cast<const ln_f32x4*>(q);
              hi[sl] = *reinterpret_cast<const ln_f32x4*>(q + 4);
            }
#pragma unroll
          for (int sl = 0; sl < xmk::kInt4MaxSplit; ++sl)
            if (sl < ks) {
#pragma unroll
              for (int e = 0; e < 4; ++e) { f[e] += lo[sl][e]; f[4 + e] += hi[sl][e]; }
            }
        };
        add_slices(p1, ks1);
        add_slices(p2, ks2);
        if (bias2) {
          Pack b2;
          b2.u = *reinterpret_cast<const ln_u32x4*>(bias2 + i);
#pragma unroll
          for (int e = 0; e < 8; ++e) f[e] += (float)b2.e[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[j].e[e] = (_Float16)f[e];
        *reinterpret_cast<ln_u32x4*>(x_out + (size_t)blockIdx.x * d + i) = v[j].u;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (float)v[j].e[e];
        s += f;
        ss += f * f;
      }
    }
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    s += __shfl_xor(s, o);
    ss += __shfl_xor(ss, o);
  }
  if ((threadIdx.x & 63) == 0) {
    s_part[0][threadIdx.x >> 6] = s;
    s_part[1][threadIdx.x >> 6] = ss;
  }
  __syncthreads();
  s = 0.f;
  ss = 0.f;
#pragma unroll
  for (int w = 0; w < LN_NT / 64; ++w) {
    s += s_part[0][w];
    ss += s_part[1][w];
  }
  const float mean = s / d;
  const float var = fmaxf(ss / d - mean * mean, 0.f);
  const float rstd = rsqrtf(var + eps);
#pragma unroll
  for (int j = 0; j < LN_MAXV; ++j) {
    const int i = (threadIdx.x + j * LN_NT) * 8;
    if (i < d) {
      Pack o;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        o.e[e] = (_Float16)(((float)v[j].e[e] - mean) * rstd * (float)gm[j].e[e] + (float)bt[j].e[e]);
      *reinterpret_cast<ln_u32x4*>(y + (size_t)blockIdx.x * d + i) = o.u;
    }
  }
}

struct Workspace {
  _Float16 *x0, *x1, *h, *qkv, *q, *attn, *ff;
  void* attn_ws;
  size_t attn_ws_bytes;
  int ks_out, ks_fc;     // K slices of out_proj and fc_out (both 1: not split)
  float *p_out, *p_fc;   // their partial sums
  size_t p_bytes;
  size_t total;
};

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

Workspace carve(const xmk_gptj_config& c, char* base) {
  Workspace w;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    char* p = base ? base + off : nullptr;
    off += align_up(bytes);
    return p;
  };
  const size_t B = (size_t)c.batch, d = (size_t)c.d_model;
  w.x0 = (_Float16*)take(B * d * 2);
  w.x1 = (_Float16*)take(B * d * 2);
  w.h = (_Float16*)take(B * d * 2);
  w.qkv = (_Float16*)take(B * 3 * d * 2);
  w.q = (_Float16*)take(B * d * 2);
  w.attn = (_Float16*)take(B * d * 2);
  w.ff = (_Float16*)take(B * (size_t)c.d_ff * 2);
  // sized for every fill level of the cache: a step attends to position + 1 <= cache_capacity keys
  w.attn_ws_bytes = xmk_fmha_decode_cache_workspace_bytes((uint32_t)c.batch, (uint32_t)c.n_head,
                                                          (uint32_t)c.head_dim, (uint32_t)c.cache_capacity);
  w.attn_ws = take(w.attn_ws_bytes);
  // fp32 partial sums of the K-split out_proj and fc_out GEMMs (when the plan splits them)
  w.ks_out = xmk::int4_plan_split(c.batch, c.d_model, c.d_model, c.group);
  w.ks_fc = xmk::int4_plan_split(c.batch, c.d_ff, c.d_model, c.group);
  if (w.ks_out < 2 || w.ks_fc < 2) w.ks_out = w.ks_fc = 1;
  w.p_bytes = (size_t)xmk::kInt4MaxSplit * 32 * d * sizeof(float);
  w.p_out = (float*)take(w.p_bytes);
  w.p_fc = (float*)take(w.p_bytes);
  w.total = off;
  return w;
}

int check_cfg(const xmk_gptj_config* c) {
  if (!c) return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: null config");
  if (c->n_layer < 1 || c->n_head < 1 || c->head_dim < 8 || c->batch < 1 || c->cache_capacity < 1 ||
      c->d_ff < 1 || c->vocab < 1)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: non-positive dimension");
  if (c->d_model != c->n_head * c->head_dim)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: d_model != n_head * head_dim");
  if (c->head_dim % 8 != 0 || c->head_dim > 256 || c->rotary_dim % 2 != 0 || c->rotary_dim > c->head_dim)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: unsupported head_dim / rotary_dim");
  if (c->d_model > LN_NT * 8 * LN_MAXV)
    return xmk::fail(XMK_UNIMPLEMENTED, "gptj_decode: d_model %d above %d", c->d_model, LN_NT * 8 * LN_MAXV);
  return XMK_OK;
}

// One int4 linear of the block as a launchable product.
int make_call(const xmk_int4_linear& l, const void* act, void* out, int64_t k, int64_t n, const xmk::Int4Epilogue& ep,
              const char* what, xmk::Int4Call* c, const xmk::Int4SplitK& split = xmk::Int4SplitK{}) {
  if (l.k != k || l.n != n)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: %s is %lldx%lld, expected %lldx%lld", what,
                     (long long)l.k, (long long)l.n, (long long)k, (long long)n);
  c->act = act; c->qweight = l.qweight; c->scales = l.scales; c->zeros = l.zeros; c->bias = l.bias; c->out = out;
  c->k = k; c->n = n; c->ep = ep; c->split = split;
  return XMK_OK;
}

}  // namespace

extern "C" size_t xmk_gptj_decode_workspace_bytes(const xmk_gptj_config* cfg) {
  if (check_cfg(cfg) != XMK_OK) return 0;
  return carve(*cfg, nullptr).total;
}

extern "C" int xmk_gptj_decode_step(const xmk_gptj_config* cfg, const xmk_gptj_layer* layers,
                                    const void* lnf_gamma, const void* lnf_beta,
                                    const xmk_int4_linear* lm_head, const void* hidden_in,
                                    int32_t position, void* logits, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  int rc = check_cfg(cfg);
  if (rc != XMK_OK) return rc;
  if (!layers || !lnf_gamma || !lnf_beta || !lm_head || !hidden_in || !logits || !workspace)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: null pointer");
  if (position < 0 || position >= cfg->cache_capacity)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: position %d outside the cache (capacity %d)",
                     position, cfg->cache_capacity);
  if (!xmk::aligned(hidden_in, 16) || !xmk::aligned(lnf_gamma, 16) || !xmk::aligned(lnf_beta, 16))
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: hidden_in and LayerNorm parameters must be 16-byte aligned");
  if (!xmk::aligned(workspace, 256)) return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: workspace must be 256-byte aligned");
  const xmk_gptj_config& c = *cfg;
  const Workspace w = carve(c, (char*)workspace);
  if (workspace_bytes < w.total)
    return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: workspace of %zu bytes, %zu needed", workspace_bytes, w.total);
  hipStream_t st = (hipStream_t)stream;
  const int64_t B = c.batch, d = c.d_model, dff = c.d_ff;
  const float scale = 1.0f / sqrtf((float)c.head_dim);
  const int64_t head_stride = (int64_t)c.cache_capacity * c.head_dim;

  // With out_proj and fc_out split over K, a block ends with x (its input) and two sets of
  // partial sums; the next LayerNorm assembles x' = x + out_proj(attn) + fc_out(...) + bias from
  // them.  Otherwise fc_out's epilogue does (out_proj's result rounded to fp16 in between).
  const _Float16* x = (const _Float16*)hidden_in;
  _Float16* xn = w.x0;
  const _Float16* pending_bias = nullptr;
  bool pending = false;
  auto run_ln = [&](const void* gamma, const void* beta) {
    if (pending) {
      hipLaunchKernelGGL(layernorm_kernel, dim3((unsigned)B), dim3(LN_NT), 0, st, x, (const _Float16*)gamma,
                         (const _Float16*)beta, w.h, (int)d, c.ln_eps, (const float*)w.p_out, w.ks_out,
                         (const float*)w.p_fc, w.ks_fc, pending_bias, xn);
      x = xn;
      xn = (xn == w.x0) ? w.x1 : w.x0;
      pending = false;
    } else {
      hipLaunchKernelGGL(layernorm_kernel, dim3((unsigned)B), dim3(LN_NT), 0, st, x, (const _Float16*)gamma,
                         (const _Float16*)beta, w.h, (int)d, c.ln_eps, (const float*)nullptr, 0, (const float*)nullptr,
                         0, (const _Float16*)nullptr, (_Float16*)nullptr);
    }
  };
  for (int l = 0; l < c.n_layer; ++l) {
    const xmk_gptj_layer& L = layers[l];
    if (!L.ln_gamma || !L.ln_beta || !L.k_cache || !L.v_cache)
      return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: layer %d has a null pointer", l);
    if (!xmk::aligned(L.ln_gamma, 16) || !xmk::aligned(L.ln_beta, 16) || !xmk::aligned(L.fc_out.bias, 16))
      return xmk::fail(XMK_INVALID_ARGUMENT, "gptj_decode: layer %d LayerNorm parameters and fc_out bias must be 16-byte aligned", l);
    run_ln(L.ln_gamma, L.ln_beta);
    // q/k/v and fc_in (+bias, gelu_new) read the same ln_1 output: one launch carries both.
    xmk::Int4Epilogue gelu;
    gelu.gelu = 1;
    xmk::Int4Call c_qkv, c_fc_in, c_out, c_fc_out;
    // The q/k/v product applies the rotary embedding and appends k and v to the caches in its epilogue.
    xmk::Int4Epilogue rope;
    rope.rope_d = (int)d; rope.head_dim = c.head_dim; rope.rotary_dim = c.rotary_dim;
    rope.capacity = c.cache_capacity; rope.position = position;
    rope.q_out = w.q; rope.k_cache = L.k_cache; rope.v_cache = L.v_cache;
    if ((rc = make_call(L.qkv, w.h, w.qkv, d, 3 * d, rope, "qkv", &c_qkv)) != XMK_OK) return rc;
    if ((rc = make_call(L.fc_in, w.h, w.ff, d, dff, gelu, "fc_in", &c_fc_in)) != XMK_OK) return rc;
    if ((rc = xmk::int4_gemm_launch2(c_qkv, &c_fc_in, B, c.group, st)) != XMK_OK) return rc;
    if ((rc = xmk_fmha_decode(w.q, L.k_cache, L.v_cache, w.attn, XMK_F16, (uint32_t)B, (uint32_t)c.n_head,
                              (uint32_t)c.head_dim, (uint32_t)(position + 1), head_stride, scale, w.attn_ws,
                              w.attn_ws_bytes, stream)) != XMK_OK)
      return rc;
    if (w.ks_out > 1 && !L.out_proj.bias) {  // (a biased out_proj takes the epilogue path)
      // out_proj(attn) and fc_out(ff) are independent: one launch, K split over work-groups, fp32
      // partial sums that the next LayerNorm adds up.
      xmk::Int4SplitK so, sf;
      so.ksplit = w.ks_out; so.partial = w.p_out; so.partial_bytes = w.p_bytes;
      sf.ksplit = w.ks_fc;  sf.partial = w.p_fc;  sf.partial_bytes = w.p_bytes;
      if ((rc = make_call(L.out_proj, w.attn, nullptr, d, d, xmk::Int4Epilogue{}, "out_proj", &c_out, so)) != XMK_OK) return rc;
      if ((rc = make_call(L.fc_out, w.ff, nullptr, dff, d, xmk::Int4Epilogue{}, "fc_out", &c_fc_out, sf)) != XMK_OK) return rc;
      if ((rc = xmk::int4_gemm_launch2(c_out, &c_fc_out, B, c.group, st)) != XMK_OK) return rc;
      pending = true;
      pending_bias = (const _Float16*)L.fc_out.bias;
    } else {
      // out_proj result goes to w.qkv's first B*d elements (the q/k/v product writes q and the caches, not this buffer);
      // fc_out adds bias, the residual x and the attention branch in its epilogue
      _Float16* a_out = w.qkv;
      if ((rc = make_call(L.out_proj, w.attn, a_out, d, d, xmk::Int4Epilogue{}, "out_proj", &c_out)) != XMK_OK) return rc;
      if ((rc = xmk::int4_gemm_launch2(c_out, nullptr, B, c.group, st)) != XMK_OK) return rc;
      xmk::Int4Epilogue res;
      res.add0 = x;
      res.add1 = a_out;
      if ((rc = make_call(L.fc_out, w.ff, xn, dff, d, res, "fc_out", &c_fc_out)) != XMK_OK) return rc;
      if ((rc = xmk::int4_gemm_launch2(c_fc_out, nullptr, B, c.group, st)) != XMK_OK) return rc;
      x = xn;
      xn = (xn == w.x0) ? w.x1 : w.x0;
    }
  }
  run_ln(lnf_gamma, lnf_beta);
  xmk::Int4Call c_head;
  if ((rc = make_call(*lm_head, w.h, logits, d, c.vocab, xmk::Int4Epilogue{}, "lm_head", &c_head)) != XMK_OK) return rc;
  if ((rc = xmk::int4_gemm_launch2(c_head, nullptr, B, c.group, st)) != XMK_OK) return rc;
  return xmk::check_launch("gptj_decode");
}
