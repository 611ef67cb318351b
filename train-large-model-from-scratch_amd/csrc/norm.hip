// RMSNorm in front of the MoE layer, fused with the bf16 cast the layer needs anyway.
//
// The reference normalises in fp32 (its `LayerNorm`, model/modules/norm.py:14-19:
// x * rsqrt(mean(x^2) + eps), cast back to the input dtype, times the weight) and hands the
// fp32 result to the MoE module, where autocast rounds it to bf16 for every product
// (model/modules/mlp.py:100, :154-155).  Here one pass reads the residual stream once and
// writes the bf16 rows the router product and the dispatch kernel consume, plus one fp32
// reciprocal RMS per row for the backward pass.  The backward kernel sums the two gradient
// contributions of the normalised rows (expert path, router path), applies the RMSNorm
// Jacobian, adds the gradient of the residual branch and reduces the weight gradient in a
// fixed order (per-block partial sums over a fixed row assignment, then a column sum), so it
// is reproducible run to run.  Both kernels are HBM-bound: each row is read once and written
// once.
#include "common.h"
#include "topk_core.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / MOE_WAVE;
constexpr int BWD_BLOCKS = 1024;  // upper bound on partial weight-gradient rows

__device__ __forceinline__ float block_sum(float v, float* red) {
#pragma unroll
  for (int o = MOE_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();  // the previous use of `red` is over
  if (lane_id() == 0) red[threadIdx.x / MOE_WAVE] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) s += red[i];
  return s;
}

template <typename T>
struct is_bf16 {
  static constexpr bool value = std::is_same<T, uint16_t>::value;
};

// NV = 16-byte column groups per thread held in registers; H8 <= NT * NV.
template <typename XT, int NV>
__global__ __launch_bounds__(NT) void rmsnorm_fwd_kernel(const XT* __restrict__ x,
                                                        const float* __restrict__ w, float eps,
                                                        int T, int H8, uint16_t* __restrict__ xn,
                                                        float* __restrict__ rstd) {
  __shared__ float red[NW];
  const int H = H8 * 8;
  Row8 wv[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < H8) wv[i] = load8(w + c * 8);
  }
  for (int t = blockIdx.x; t < T; t += gridDim.x) {
    Row8 xv[NV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < H8) {
        xv[i] = load8(x + (size_t)t * H + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += xv[i].v[j] * xv[i].v[j];
      }
    }
    ss = block_sum(ss, red);
    const float r = rsqrtf(ss / (float)H + eps);
    if (threadIdx.x == 0) rstd[t] = r;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < H8) {
        Row8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float v = xv[i].v[j] * r;
          if (is_bf16<XT>::value) v = bf16_to_f32(f32_to_bf16(v));  // `.to(input_dtype)`, norm.py:19
          o.v[j] = wv[i].v[j] * v;
        }
        store8(xn + (size_t)t * H + c * 8, o);
      }
    }
  }
}

// The normalisation with the router behind it (model/gpt.py:32 into model/modules/mlp.py:100-103
// in one pass): a block normalises RB rows, keeps their bf16 form in LDS besides writing it out,
// multiplies them with the router weight on the matrix cores (v_mfma_f32_16x16x32_bf16: rows =
// tokens from LDS, columns = experts straight from L2, the four waves split the contraction and
// add their partial products through LDS), rounds the logits to bf16 (what the layer returns and
// selects on) and runs the wave-level top-k + softmax on them.  The normalised rows are not read
// again for the router, and the logits never leave the chip before selection.
constexpr int RB = 16;       // rows (tokens) per block
constexpr int RMAX_EB = 8;   // 16-expert column blocks: E <= 128

template <typename XT, int NV>
__global__ __launch_bounds__(NT) void rmsnorm_router_fwd_kernel(
    const XT* __restrict__ x, const float* __restrict__ w, float eps, int T, int H8,
    const uint16_t* __restrict__ wr, int E, int k, uint16_t* __restrict__ xn, float* __restrict__ rstd,
    uint16_t* __restrict__ logits, int32_t* __restrict__ ids, float* __restrict__ gates) {
  extern __shared__ __attribute__((aligned(16))) uint16_t rows[];  // [RB][H + 8]; later fp32 partials
  __shared__ float red[NW];
  __shared__ uint16_t lg16[RB * RMAX_EB * 16];
  const int H = H8 * 8, LDT = H + 8;
  const int lane = lane_id(), wv = threadIdx.x / MOE_WAVE;
  const int t0 = blockIdx.x * RB;
  Row8 wv8[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < H8) wv8[i] = load8(w + c * 8);
  }
  for (int rr = 0; rr < RB; ++rr) {
    const int t = t0 + rr;
    if (t >= T) {  // block-uniform: rows past the end are zero rows for the product
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * NT;
        if (c < H8) *reinterpret_cast<u32x4*>(rows + rr * LDT + c * 8) = u32x4{0, 0, 0, 0};
      }
      continue;
    }
    Row8 xv[NV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < H8) {
        xv[i] = load8(x + (size_t)t * H + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += xv[i].v[j] * xv[i].v[j];
      }
    }
    ss = block_sum(ss, red);
    const float r = rsqrtf(ss / (float)H + eps);
    if (threadIdx.x == 0) rstd[t] = r;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < H8) {
        Row8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float v = xv[i].v[j] * r;
          if (is_bf16<XT>::value) v = bf16_to_f32(f32_to_bf16(v));  // `.to(input_dtype)`, norm.py:19
          o.v[j] = wv8[i].v[j] * v;
        }
        store8(xn + (size_t)t * H + c * 8, o);
        store8(rows + rr * LDT + c * 8, o);
      }
    }
  }
  __syncthreads();
  // logits[m][e] = sum_h rows[m][h] * wr[e][h]: lane l holds A row l % 16 (token) and B row
  // l % 16 of the column block (expert), 8 consecutive h at (l / 16) * 8 of the 32-wide k-step
  const int EB = E / 16;
  f32x4 acc[RMAX_EB];
#pragma unroll
  for (int nb = 0; nb < RMAX_EB; ++nb) acc[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const int l16 = lane & 15, lq = lane >> 4;
  for (int ks = wv; ks < H / 32; ks += NW) {
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(rows + l16 * LDT + ks * 32 + lq * 8);
#pragma unroll
    for (int nb = 0; nb < RMAX_EB; ++nb) {
      if (nb < EB) {
        const bf16x8 b = *reinterpret_cast<const bf16x8*>(wr + (size_t)(nb * 16 + l16) * H + ks * 32 + lq * 8);
        acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[nb], 0, 0, 0);
      }
    }
  }
  __syncthreads();  // every wave is done with the rows: their memory takes the partial products
  float* part = reinterpret_cast<float*>(rows);  // [NW][RB][E]
  // accumulator layout: lane l holds column l % 16 (expert) of rows 4 * (l / 16) .. + 3 (tokens)
#pragma unroll
  for (int nb = 0; nb < RMAX_EB; ++nb) {
    if (nb < EB) {
#pragma unroll
      for (int i = 0; i < 4; ++i) part[(wv * RB + lq * 4 + i) * E + nb * 16 + l16] = acc[nb][i];
    }
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < RB * E; idx += NT) {
    float v = 0.f;
#pragma unroll
    for (int q = 0; q < NW; ++q) v += part[q * RB * E + idx];  // fixed order: reproducible
    const uint16_t b = f32_to_bf16(v);
    lg16[idx] = b;
    const int m = idx / E;
    if (t0 + m < T) logits[(size_t)(t0 + m) * E + (idx - m * E)] = b;
  }
  __syncthreads();
  // selection: one wave per token
  for (int m = wv; m < RB; m += NW) {
    const int t = t0 + m;
    if (t >= T) break;
    uint64_t key[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int e = i * MOE_WAVE + lane;
      key[i] = e < E ? moe_topk_key(bf16_to_f32(lg16[m * E + e]), e) : 0;
    }
    int my_id;
    float my_gate;
    moe_topk_softmax_wave<2>(key, k, lane, my_id, my_gate);
    if (lane < k) {
      ids[(size_t)t * k + lane] = my_id;
      gates[(size_t)t * k + lane] = my_gate;
    }
  }
}

// dx[t] = dres[t] + rstd * (w*g - xhat * mean(w*g*xhat)),  g = d1[t] + d2[t],  xhat = x*rstd;
// part[block] = sum over the block's rows of g*xhat.
template <typename XT, typename DT, int NV>
__global__ __launch_bounds__(NT) void rmsnorm_bwd_kernel(
    const XT* __restrict__ x, const float* __restrict__ w, const float* __restrict__ rstd,
    const DT* __restrict__ d1, const uint16_t* __restrict__ d2, const XT* __restrict__ dres, int T,
    int H8, XT* __restrict__ dx, float* __restrict__ part) {
  __shared__ float red[NW];
  const int H = H8 * 8;
  Row8 wv[NV], dwv[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < H8) wv[i] = load8(w + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) dwv[i].v[j] = 0.f;
  }
  for (int t = blockIdx.x; t < T; t += gridDim.x) {
    const float r = rstd[t];
    Row8 xh[NV], gw[NV];
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < H8) {
        const size_t at = (size_t)t * H + c * 8;
        xh[i] = load8(x + at);
        Row8 g = load8(d1 + at);
        if (d2) {
          const Row8 g2 = load8(d2 + at);
#pragma unroll
          for (int j = 0; j < 8; ++j) g.v[j] += g2.v[j];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          xh[i].v[j] *= r;
          dwv[i].v[j] += g.v[j] * xh[i].v[j];
          gw[i].v[j] = g.v[j] * wv[i].v[j];
          dot += gw[i].v[j] * xh[i].v[j];
        }
      }
    }
    dot = block_sum(dot, red);
    const float m = dot / (float)H;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = threadIdx.x + i * NT;
      if (c < H8) {
        const size_t at = (size_t)t * H + c * 8;
        Row8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o.v[j] = r * (gw[i].v[j] - xh[i].v[j] * m);
        if (dres) {
          const Row8 a = load8(dres + at);
#pragma unroll
          for (int j = 0; j < 8; ++j) o.v[j] += a.v[j];
        }
        store8(dx + at, o);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < H8) store8(part + (size_t)blockIdx.x * H + c * 8, dwv[i]);
  }
}

// dw[c] = sum_b part[b][c], b ascending within each of the block's NW row groups, groups
// combined in ascending order: one fixed order whatever the launch.
__global__ __launch_bounds__(NT) void colsum_kernel(const float* __restrict__ part, int nb, int H,
                                                   float* __restrict__ dw) {
  __shared__ float red[NW][MOE_WAVE];
  const int c = blockIdx.x * MOE_WAVE + lane_id(), g = threadIdx.x / MOE_WAVE;
  const int per = (nb + NW - 1) / NW;
  float s = 0.f;
  if (c < H)
    for (int b = g * per; b < nb && b < (g + 1) * per; ++b) s += part[(size_t)b * H + c];
  red[g][lane_id()] = s;
  __syncthreads();
  if (g == 0 && c < H) {
    float tot = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) tot += red[i][lane_id()];
    dw[c] = tot;
  }
}

inline int bwd_blocks(int64_t T) { return (int)(T < BWD_BLOCKS ? (T < 1 ? 1 : T) : BWD_BLOCKS); }

inline int pick_nv(int64_t H) {
  const int64_t need = (H / 8 + NT - 1) / NT;
  return need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : 0;  // H <= 8192
}

template <typename XT>
int launch_fwd(const void* x, const float* w, float eps, int64_t T, int64_t H, uint16_t* xn,
               float* rstd, hipStream_t s) {
  const dim3 grid((unsigned)(T < 256 * 16 ? T : 256 * 16)), block(NT);
#define MOE_NORM_FWD(NV)                                                                          \
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<XT, NV>), grid, block, 0, s, (const XT*)x, w, eps, (int)T, \
                     (int)(H / 8), xn, rstd)
  switch (pick_nv(H)) {
    case 1: MOE_NORM_FWD(1); break;
    case 2: MOE_NORM_FWD(2); break;
    case 4: MOE_NORM_FWD(4); break;
    default: return MOE_ERR_LIMIT;
  }
#undef MOE_NORM_FWD
  return moe_launch_status();
}

template <typename XT, typename DT>
int launch_bwd(const void* x, const float* w, const float* rstd, const void* d1, const uint16_t* d2,
               const void* dres, int64_t T, int64_t H, void* dx, float* part, hipStream_t s) {
  const dim3 grid((unsigned)bwd_blocks(T)), block(NT);
#define MOE_NORM_BWD(NV)                                                                       \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<XT, DT, NV>), grid, block, 0, s, (const XT*)x, w, rstd, \
                     (const DT*)d1, d2, (const XT*)dres, (int)T, (int)(H / 8), (XT*)dx, part)
  switch (pick_nv(H)) {
    case 1: MOE_NORM_BWD(1); break;
    case 2: MOE_NORM_BWD(2); break;
    case 4: MOE_NORM_BWD(4); break;
    default: return MOE_ERR_LIMIT;
  }
#undef MOE_NORM_BWD
  return moe_launch_status();
}

int check_norm(int64_t T, int64_t H) {
  if (T < 0 || H <= 0 || (H % 8) != 0) return MOE_ERR_SHAPE;
  if (T > (int64_t)1 << 30 || pick_nv(H) == 0) return MOE_ERR_LIMIT;
  return 0;
}

}  // namespace

extern "C" int moe_rmsnorm_fwd(const void* x, int x_dtype, const float* weight, float eps, int64_t T,
                               int64_t H, uint16_t* xn, float* rstd, void* stream) {
  if (int rc = check_norm(T, H)) return rc;
  if (T == 0) return 0;
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(weight);
  MOE_CHECK_PTR(xn);
  if (!rstd) return MOE_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  if (x_dtype == MOE_DT_BF16) return launch_fwd<uint16_t>(x, weight, eps, T, H, xn, rstd, s);
  if (x_dtype == MOE_DT_F32) return launch_fwd<float>(x, weight, eps, T, H, xn, rstd, s);
  return MOE_ERR_DTYPE;
}

extern "C" int moe_rmsnorm_router_supported(int64_t H, int64_t E, int64_t k) {
  return (H > 0 && E > 0 && k > 0 && (H % 32) == 0 && H <= 4096 && (E % 16) == 0 && E <= 16 * RMAX_EB && k <= E &&
          k <= MOE_MAX_TOPK)
             ? 1 : 0;
}

extern "C" int moe_rmsnorm_router_fwd(const void* x, int x_dtype, const float* weight, float eps,
                                      const uint16_t* router_weight, int64_t T, int64_t H, int64_t E,
                                      int64_t k, uint16_t* xn, float* rstd, uint16_t* logits,
                                      int32_t* ids, float* gates, void* stream) {
  if (int rc = check_norm(T, H)) return rc;
  if (E <= 0 || k <= 0 || k > E) return MOE_ERR_SHAPE;
  if (!moe_rmsnorm_router_supported(H, E, k)) return MOE_ERR_LIMIT;
  if (T == 0) return 0;
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(weight);
  MOE_CHECK_PTR(router_weight);
  MOE_CHECK_PTR(xn);
  if (!rstd || !logits || !ids || !gates) return MOE_ERR_NULL;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((unsigned)((T + RB - 1) / RB)), block(NT);
  const size_t lds = (size_t)RB * (H + 8) * 2 > (size_t)NW * RB * E * 4 ? (size_t)RB * (H + 8) * 2 : (size_t)NW * RB * E * 4;
  constexpr int MAX_ROUTER_LDS = RB * (4096 + 8) * 2 > NW * RB * 16 * RMAX_EB * 4 ? RB * (4096 + 8) * 2 : NW * RB * 16 * RMAX_EB * 4;
  if (lds > (size_t)MAX_ROUTER_LDS) return MOE_ERR_LIMIT;
#define MOE_NORM_ROUTER(XT, NV)                                                                          \
  do {                                                                                                   \
    auto kern = rmsnorm_router_fwd_kernel<XT, NV>;                                                       \
    static bool attr_done[MOE_MAX_DEVICES]; /* per GPU and instantiation: set once, to the largest */    \
    const int dev = moe_current_device();   /* footprint any supported shape asks for              */    \
    if (!attr_done[dev]) {                                                                               \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,  \
                                         MAX_ROUTER_LDS);                                                \
      if (e != hipSuccess) return (int)e;                                                                \
      attr_done[dev] = true;                                                                             \
    }                                                                                                    \
    hipLaunchKernelGGL(kern, grid, block, lds, s, (const XT*)x, weight, eps, (int)T, (int)(H / 8),       \
                       router_weight, (int)E, (int)k, xn, rstd, logits, ids, gates);                     \
  } while (0)
  const int nv = pick_nv(H);
  if (x_dtype == MOE_DT_BF16) {
    if (nv == 1) MOE_NORM_ROUTER(uint16_t, 1); else MOE_NORM_ROUTER(uint16_t, 2);
  } else if (x_dtype == MOE_DT_F32) {
    if (nv == 1) MOE_NORM_ROUTER(float, 1); else MOE_NORM_ROUTER(float, 2);
  } else {
    return MOE_ERR_DTYPE;
  }
#undef MOE_NORM_ROUTER
  return moe_launch_status();
}

extern "C" int64_t moe_rmsnorm_bwd_workspace_bytes(int64_t T, int64_t H) {
  if (T < 0 || H <= 0) return 0;
  return (int64_t)bwd_blocks(T) * H * (int64_t)sizeof(float);
}

extern "C" int moe_rmsnorm_bwd(const void* x, int x_dtype, const float* weight, const float* rstd,
                               const void* d1, int d1_dtype, const uint16_t* d2, const void* dres,
                               int64_t T, int64_t H, void* dx, float* dweight, void* workspace,
                               int64_t workspace_bytes, void* stream) {
  if (int rc = check_norm(T, H)) return rc;
  MOE_CHECK_PTR(dweight);
  hipStream_t s = (hipStream_t)stream;
  if (T == 0) {  // no rows: the weight gradient is zero
    hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((H + MOE_WAVE - 1) / MOE_WAVE)), dim3(NT), 0, s,
                       (const float*)dweight, 0, (int)H, dweight);
    return moe_launch_status();
  }
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(weight);
  MOE_CHECK_PTR(d1);
  MOE_CHECK_PTR(dx);
  MOE_CHECK_PTR(workspace);
  if (!rstd) return MOE_ERR_NULL;
  if (d2 && !aligned16(d2)) return MOE_ERR_ALIGN;
  if (dres && !aligned16(dres)) return MOE_ERR_ALIGN;
  if (workspace_bytes < moe_rmsnorm_bwd_workspace_bytes(T, H)) return MOE_ERR_WORKSPACE;
  float* part = (float*)workspace;
  int rc;
  if (x_dtype == MOE_DT_BF16 && d1_dtype == MOE_DT_BF16)
    rc = launch_bwd<uint16_t, uint16_t>(x, weight, rstd, d1, d2, dres, T, H, dx, part, s);
  else if (x_dtype == MOE_DT_BF16 && d1_dtype == MOE_DT_F32)
    rc = launch_bwd<uint16_t, float>(x, weight, rstd, d1, d2, dres, T, H, dx, part, s);
  else if (x_dtype == MOE_DT_F32 && d1_dtype == MOE_DT_BF16)
    rc = launch_bwd<float, uint16_t>(x, weight, rstd, d1, d2, dres, T, H, dx, part, s);
  else if (x_dtype == MOE_DT_F32 && d1_dtype == MOE_DT_F32)
    rc = launch_bwd<float, float>(x, weight, rstd, d1, d2, dres, T, H, dx, part, s);
  else
    return MOE_ERR_DTYPE;
  if (rc) return rc;
  hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((H + MOE_WAVE - 1) / MOE_WAVE)), dim3(NT), 0, s,
                     (const float*)part, bwd_blocks(T), (int)H, dweight);
  return moe_launch_status();
}
