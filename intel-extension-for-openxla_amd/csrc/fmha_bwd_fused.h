// Interface of the fused attention backward kernels (fmha_bwd_fused.hip) for the entry point in
// fmha_bwd.hip.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace fmha_bwd_fused {

struct Args {
  const void* q;
  const void* k;
  const void* v;
  const void* d_o;
  const void* bias;   // [units, F, T] additive bias or null
  const float* lse;   // [units, F] log-sum-exp of the forward pass times log2(e)
  const float* dsum;  // [units, F] rowsum(dO o O)
  void* dq;
  void* dk;
  void* dv;
  int H, F, T;
  float scale;
  bool causal;
};

// Head sizes up to 256 (multiples of 8); a bias of at most 2 GiB per unit.
bool eligible(const Args& a, uint64_t units);
// Two launches: keys own (dK, dV), then queries own (dQ).
void launch(const Args& a, uint64_t units, bool bf16, hipStream_t stream);

}  // namespace fmha_bwd_fused
