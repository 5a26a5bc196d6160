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
  const void* o;         // [units, F, H] output of the forward pass
  const void* bias;      // [units, F, T] additive bias or null
  const float* lse_fwd;  // [units, F] log-sum-exp of the forward pass
  float* lse;            // scratch [units, F]: LSE times log2(e)       } written by the queries-own launch,
  float* dsum;           // scratch [units, F]: D = rowsum(dO o O)       } read by the keys-own launches after it
  void* dq;
  void* dk;
  void* dv;
  int H, F, T;
  float scale;
  bool causal;
};

// Head sizes up to 256 (multiples of 8); a bias of at most 2 GiB per unit.
bool eligible(const Args& a, uint64_t units);
// Queries own (dQ; it also forms the two per-row statistics), then keys own (dK, dV).
void launch(const Args& a, uint64_t units, bool bf16, hipStream_t stream);

}  // namespace fmha_bwd_fused
