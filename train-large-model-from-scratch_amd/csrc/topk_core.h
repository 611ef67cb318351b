// Wave-level top-k + softmax over the k winners, shared by the router kernel and the fused
// norm + router kernel.  One 64-lane wavefront owns one token; expert e lives in lane e % 64,
// slot e / 64.
#pragma once
#include "common.h"

__device__ __forceinline__ uint32_t moe_orderable(float v) {
  v += 0.0f;  // -0.0 -> +0.0 so that the two compare equal, as they do for torch.topk
  uint32_t u = __builtin_bit_cast(uint32_t, v);
  // a NaN of either sign ranks above every number, as it does for torch.topk (and maps back
  // to a NaN, so the token's gates are NaN as the reference's are)
  return (v != v) ? 0xffffffffu : u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float moe_from_orderable(uint32_t u) {
  u ^= ((u >> 31) ? 0x80000000u : 0xffffffffu);
  return __builtin_bit_cast(float, u);
}
// key = (orderable(logit) << 32) | (0xffffffff - expert): the maximum key is the largest logit
// and, among equal logits, the smallest expert index.  0 marks "taken / absent".
__device__ __forceinline__ uint64_t moe_topk_key(float logit, int expert) {
  return ((uint64_t)moe_orderable(logit) << 32) | (uint64_t)(0xffffffffu - (uint32_t)expert);
}

// Wave-wide maximum of a 64-bit key, the same value in every lane.  Four exchange steps inside
// each row of 16 lanes go through the DPP data path of the vector ALU (neighbour, pair, mirrored
// half row, mirrored row: no LDS, no waits), then the four row maxima are read as scalars.
template <int CTRL>
__device__ __forceinline__ uint64_t moe_dpp_max_step(uint64_t v) {
  const int lo = (int)(uint32_t)v, hi = (int)(uint32_t)(v >> 32);
  const uint32_t lo2 = (uint32_t)__builtin_amdgcn_update_dpp(0, lo, CTRL, 0xf, 0xf, false);
  const uint32_t hi2 = (uint32_t)__builtin_amdgcn_update_dpp(0, hi, CTRL, 0xf, 0xf, false);
  const uint64_t o = ((uint64_t)hi2 << 32) | lo2;
  return o > v ? o : v;
}
__device__ __forceinline__ uint64_t moe_wave_max_u64(uint64_t v) {
  v = moe_dpp_max_step<0xB1>(v);   // quad_perm [1,0,3,2]: lane ^ 1
  v = moe_dpp_max_step<0x4E>(v);   // quad_perm [2,3,0,1]: lane ^ 2
  v = moe_dpp_max_step<0x141>(v);  // row_half_mirror: the other quad of each 8 lanes
  v = moe_dpp_max_step<0x140>(v);  // row_mirror: the other half of each 16 lanes
  const int lo = (int)(uint32_t)v, hi = (int)(uint32_t)(v >> 32);
  uint64_t best = 0;
#pragma unroll
  for (int row = 0; row < MOE_WAVE / 16; ++row) {
    const uint64_t o = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane(hi, 16 * row) << 32) |
                       (uint32_t)__builtin_amdgcn_readlane(lo, 16 * row);
    best = o > best ? o : best;
  }
  return best;
}
__device__ __forceinline__ float moe_wave_sum_f32(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, MOE_WAVE);
  return v;
}

// k rounds of a wave-wide maximum over the keys (consumed), then the softmax over the k selected
// logits in fp32.  On return lane j < k holds slot j: expert id and gate.
template <int VPL>
__device__ __forceinline__ void moe_topk_softmax_wave(uint64_t (&key)[VPL], int k, int lane, int& my_id,
                                                      float& my_gate) {
  my_id = 0;
  float my_val = 0.f;
  for (int j = 0; j < k; ++j) {
    uint64_t best = key[0];
#pragma unroll
    for (int i = 1; i < VPL; ++i) best = key[i] > best ? key[i] : best;
    best = moe_wave_max_u64(best);
    const uint32_t e = 0xffffffffu - (uint32_t)best;
#pragma unroll
    for (int i = 0; i < VPL; ++i)
      if ((int)e == i * MOE_WAVE + lane) key[i] = 0;
    if (lane == j) {
      my_id = (int)e;
      my_val = moe_from_orderable((uint32_t)(best >> 32));
    }
  }
  const float vmax = __shfl(my_val, 0, MOE_WAVE);
  const float p = lane < k ? expf(my_val - vmax) : 0.f;
  const float s = moe_wave_sum_f32(p);
  my_gate = p / s;
}
