// Router top-k + softmax (forward and backward) for gfx950.
//
// One 64-lane wavefront owns one token.  The E logits of the token are spread over the
// lanes (expert e lives in lane e%64, slot e/64), selection is k rounds of a wave-wide
// max-reduction over 64-bit keys, and the softmax over the k winners is a wave reduction.
// HBM-bound: reads T*E logits, writes T*k ids and gates.
#include "common.h"
#include "topk_core.h"

namespace {

template <int VPL, typename LT>
__global__ __launch_bounds__(256) void router_topk_fwd_kernel(const LT* __restrict__ logits,
                                                             const float* __restrict__ bias,
                                                             int T, int E, int k,
                                                             int32_t* __restrict__ ids,
                                                             float* __restrict__ gates) {
  const int lane = lane_id();
  const int t = blockIdx.x * (blockDim.x / MOE_WAVE) + (threadIdx.x / MOE_WAVE);
  if (t >= T) return;  // whole wave exits together
  uint64_t key[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = i * MOE_WAVE + lane;
    key[i] = 0;
    if (e < E) {
      float v;
      if constexpr (sizeof(LT) == 2) v = bf16_to_f32(((const uint16_t*)logits)[(size_t)t * E + e]);
      else v = ((const float*)logits)[(size_t)t * E + e];
      if (bias) v += bias[e];
      key[i] = moe_topk_key(v, e);
    }
  }
  int my_id;
  float my_gate;
  moe_topk_softmax_wave<VPL>(key, k, lane, my_id, my_gate);
  if (lane < k) {
    ids[(size_t)t * k + lane] = my_id;
    gates[(size_t)t * k + lane] = my_gate;
  }
}

template <int VPL, typename DT>
__global__ __launch_bounds__(256) void router_topk_bwd_kernel(const float* __restrict__ gates,
                                                             const float* __restrict__ dgates,
                                                             const int32_t* __restrict__ ids,
                                                             int T, int E, int k,
                                                             DT* __restrict__ dlogits) {
  const int lane = lane_id();
  const int t = blockIdx.x * (blockDim.x / MOE_WAVE) + (threadIdx.x / MOE_WAVE);
  if (t >= T) return;
  float g = 0.f, dg = 0.f;
  int id = -1;
  if (lane < k) {
    g = gates[(size_t)t * k + lane];
    dg = dgates[(size_t)t * k + lane];
    id = ids[(size_t)t * k + lane];
  }
  const float s = moe_wave_sum_f32(g * dg);
  const float dsel = g * (dg - s);
  float val[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) val[i] = 0.f;
  for (int j = 0; j < k; ++j) {
    const int idj = __shfl(id, j, MOE_WAVE);
    const float dj = __shfl(dsel, j, MOE_WAVE);
#pragma unroll
    for (int i = 0; i < VPL; ++i)
      if (idj == i * MOE_WAVE + lane) val[i] = dj;
  }
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    const int e = i * MOE_WAVE + lane;
    if (e < E) {
      if constexpr (sizeof(DT) == 2) ((uint16_t*)dlogits)[(size_t)t * E + e] = f32_to_bf16(val[i]);
      else ((float*)dlogits)[(size_t)t * E + e] = val[i];
    }
  }
}

template <typename F>
int dispatch_vpl(int64_t E, F&& f) {
  if (E <= 64) return f(std::integral_constant<int, 1>{});
  if (E <= 128) return f(std::integral_constant<int, 2>{});
  if (E <= 256) return f(std::integral_constant<int, 4>{});
  return f(std::integral_constant<int, 8>{});
}

}  // namespace

extern "C" int moe_router_topk_fwd(const void* logits, int logits_dtype, const float* bias,
                                   int64_t T, int64_t E, int64_t k, int32_t* ids_out,
                                   float* gates_out, void* stream) {
  if (T < 0 || E <= 0 || k <= 0 || k > E) return MOE_ERR_SHAPE;
  if (E > MOE_MAX_EXPERTS || k > MOE_MAX_TOPK || T > (int64_t)1 << 30) return MOE_ERR_LIMIT;
  if (logits_dtype != MOE_DT_BF16 && logits_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  if (T == 0) return 0;  // nothing to read or write: empty buffers may be null
  if (!logits || !ids_out || !gates_out) return MOE_ERR_NULL;
  const dim3 block(256), grid((unsigned)((T + 3) / 4));
  hipStream_t s = (hipStream_t)stream;
  return dispatch_vpl(E, [&](auto vpl) {
    constexpr int V = decltype(vpl)::value;
    if (logits_dtype == MOE_DT_BF16)
      hipLaunchKernelGGL((router_topk_fwd_kernel<V, uint16_t>), grid, block, 0, s,
                         (const uint16_t*)logits, bias, (int)T, (int)E, (int)k, ids_out, gates_out);
    else
      hipLaunchKernelGGL((router_topk_fwd_kernel<V, float>), grid, block, 0, s,
                         (const float*)logits, bias, (int)T, (int)E, (int)k, ids_out, gates_out);
    return moe_launch_status();
  });
}

extern "C" int moe_router_topk_bwd(const float* gates, const float* dgates, const int32_t* ids,
                                   int64_t T, int64_t E, int64_t k, void* dlogits,
                                   int dlogits_dtype, void* stream) {
  if (T < 0 || E <= 0 || k <= 0 || k > E) return MOE_ERR_SHAPE;
  if (E > MOE_MAX_EXPERTS || k > MOE_MAX_TOPK || T > (int64_t)1 << 30) return MOE_ERR_LIMIT;
  if (dlogits_dtype != MOE_DT_BF16 && dlogits_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  if (T == 0) return 0;
  if (!gates || !dgates || !ids || !dlogits) return MOE_ERR_NULL;
  const dim3 block(256), grid((unsigned)((T + 3) / 4));
  hipStream_t s = (hipStream_t)stream;
  return dispatch_vpl(E, [&](auto vpl) {
    constexpr int V = decltype(vpl)::value;
    if (dlogits_dtype == MOE_DT_BF16)
      hipLaunchKernelGGL((router_topk_bwd_kernel<V, uint16_t>), grid, block, 0, s, gates, dgates,
                         ids, (int)T, (int)E, (int)k, (uint16_t*)dlogits);
    else
      hipLaunchKernelGGL((router_topk_bwd_kernel<V, float>), grid, block, 0, s, gates, dgates, ids,
                         (int)T, (int)E, (int)k, (float*)dlogits);
    return moe_launch_status();
  });
}
