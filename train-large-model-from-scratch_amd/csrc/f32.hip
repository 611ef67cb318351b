// The expert path in fp32, for callers that run the layer without autocast on fp32 tensors: the
// reference then computes its three bmm's, SwiGLU, gate weighting and k-sum in fp32
// (model/modules/mlp.py:133-169 with fp32 operands), and so does this file.  Same routing and
// dispatch kernels as the bf16 path; what differs is the row type of the expert-contiguous
// buffers (fp32 [R,H] / [R,I]) and the matrix instruction (v_mfma_f32_32x32x2_f32, fp32
// operands, fp32 accumulate).  A compatibility mode: correct and bounds-checked, 64 x 64 or
// 128 x 128 tiles from plain HIP, 75 to 80 % of the fp32 matrix peak on large shapes.
#include "common.h"

namespace {

constexpr int TK = 16;  // depth of a k-tile

// Output tiles of T x T (T = 64 or 128) per workgroup of four waves (2 x 2, each T/2 x T/2 as
// NB x NB blocks of 32 x 32).  LDS tiles are k-major: row = k, T values of m (or n) + 4 of padding.
template <int T>
struct Shape {
  static constexpr int LD = T + 4;
  static constexpr int NB = T / 64;   // 32 x 32 blocks per wave and dimension
  static constexpr int PER = T / 64;  // 16-byte loads per thread, operand and k-tile
};

struct F32Gemm {
  const float* A;
  const float* B;
  float* C;
  const int32_t* offs;
  int E, R;
  int M, N, K;  // row-ragged: N output columns, K depth.  k-ragged: M x N outputs per expert.
  int accumulate;
};

// T x 16 tile of an operand whose k index is contiguous in memory (element (i, k) at
// base[i * ld + k]): a thread takes one row (+64) and four consecutive k values, and writes them
// transposed into the k-major LDS tile.
// Which row and which k quad of a T x 16 tile thread t takes: lanes 2n and 2n+1 of a half-wave take
// the two k quads 0,1 (lower half-wave) or 2,3 (upper) of row n, so that the 32 lanes the LDS serves
// together write their transposed values to 32 different banks (16 rows x 2 quads, rows of
// 4 * LD bytes with LD = 4 mod 32).
__device__ __forceinline__ int kcont_row() { return ((threadIdx.x >> 1) & 15) + 16 * (threadIdx.x >> 6); }
__device__ __forceinline__ int kcont_quad() { return (threadIdx.x & 1) + 2 * ((threadIdx.x >> 5) & 1); }

template <int T>
__device__ __forceinline__ void load_kcont(f32x4 (&v)[Shape<T>::PER], const float* base, long long ld, int i0,
                                           int i_lim, int k0, int K) {
  const int k = k0 + kcont_quad() * 4;
#pragma unroll
  for (int r = 0; r < Shape<T>::PER; ++r) {
    const int i = i0 + kcont_row() + 64 * r;
    v[r] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (i < i_lim && k < K) v[r] = *reinterpret_cast<const f32x4*>(base + (long long)i * ld + k);  // (K % 4 == 0)
  }
}
template <int T>
__device__ __forceinline__ void stage_kcont(float* s, const f32x4 (&v)[Shape<T>::PER]) {
  const int k = kcont_quad() * 4;
#pragma unroll
  for (int r = 0; r < Shape<T>::PER; ++r) {
    const int i = kcont_row() + 64 * r;
#pragma unroll
    for (int x = 0; x < 4; ++x) s[(k + x) * Shape<T>::LD + i] = v[r][x];
  }
}
// 16 x T tile of an operand whose m (or n) index is contiguous (element (k, i) at
// base[k * ld + i]): T/4 threads per k row take four values each, 1024/T k rows per pass.
template <int T>
__device__ __forceinline__ void load_icont(f32x4 (&v)[Shape<T>::PER], const float* base, long long ld, int k0,
                                           int k_lim, int i0, int i_lim) {
  const int i = i0 + (threadIdx.x % (T / 4)) * 4;
#pragma unroll
  for (int r = 0; r < Shape<T>::PER; ++r) {
    const int k = k0 + threadIdx.x / (T / 4) + (1024 / T) * r;
    v[r] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (k < k_lim && i < i_lim) v[r] = *reinterpret_cast<const f32x4*>(base + (long long)k * ld + i);  // (i_lim % 4 == 0)
  }
}
template <int T>
__device__ __forceinline__ void stage_icont(float* s, const f32x4 (&v)[Shape<T>::PER]) {
#pragma unroll
  for (int r = 0; r < Shape<T>::PER; ++r)
    *reinterpret_cast<f32x4*>(s + (threadIdx.x / (T / 4) + (1024 / T) * r) * Shape<T>::LD +
                              (threadIdx.x % (T / 4)) * 4) = v[r];
}

// One k-tile of 16 from LDS.  The operands go in swapped, so that a lane ends up with row
// lane%32 of a 32 x 32 block and four consecutive columns per group of four accumulator
// registers (columns 8g + 4*(lane/32) .. +3).
template <int T>
__device__ __forceinline__ void mma_tile(const float* sA, const float* sB, int wm, int wn,
                                         f32x16 (&acc)[Shape<T>::NB][Shape<T>::NB]) {
  constexpr int NB = Shape<T>::NB, LD = Shape<T>::LD;
  const int l32 = threadIdx.x & 31, lh = (threadIdx.x >> 5) & 1;
#pragma unroll
  for (int kk = 0; kk < TK / 2; ++kk) {
    float a[NB], b[NB];
#pragma unroll
    for (int x = 0; x < NB; ++x) {
      a[x] = sA[(2 * kk + lh) * LD + (wm * NB + x) * 32 + l32];
      b[x] = sB[(2 * kk + lh) * LD + (wn * NB + x) * 32 + l32];
    }
#pragma unroll
    for (int bi = 0; bi < NB; ++bi)
#pragma unroll
      for (int bj = 0; bj < NB; ++bj)
        acc[bi][bj] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[bj], a[bi], acc[bi][bj], 0, 0, 0);
  }
}

template <int T>
__device__ __forceinline__ void store_tile(float* C, long long ldc, int m0, int m_lim, int n0, int n_lim, int wm,
                                           int wn, const f32x16 (&acc)[Shape<T>::NB][Shape<T>::NB],
                                           bool accumulate) {
  constexpr int NB = Shape<T>::NB;
  const int l32 = threadIdx.x & 31, lh = (threadIdx.x >> 5) & 1;
#pragma unroll
  for (int bi = 0; bi < NB; ++bi) {
    const int m = m0 + (wm * NB + bi) * 32 + l32;
    if (m >= m_lim) continue;
#pragma unroll
    for (int bj = 0; bj < NB; ++bj)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + (wn * NB + bj) * 32 + 8 * g + 4 * lh;
        if (n >= n_lim) continue;  // (n_lim % 4 == 0: the four columns are inside or outside together)
        f32x4* dst = reinterpret_cast<f32x4*>(C + (long long)m * ldc + n);
        f32x4 v = {acc[bi][bj][4 * g], acc[bi][bj][4 * g + 1], acc[bi][bj][4 * g + 2], acc[bi][bj][4 * g + 3]};
        if (accumulate) v += *dst;
        *dst = v;
      }
  }
}

template <int T>
__device__ __forceinline__ void clear(f32x16 (&acc)[Shape<T>::NB][Shape<T>::NB]) {
#pragma unroll
  for (int bi = 0; bi < Shape<T>::NB; ++bi)
#pragma unroll
    for (int bj = 0; bj < Shape<T>::NB; ++bj)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[bi][bj][i] = 0.f;
}

// Row-ragged: C[r, :] (+)= A[r, :] x B_e for the rows r of expert e.  A [R,K] row-major;
// B_e = B + e*N*K holds either [N,K] (B_KCONT: C = A B_e^T, the forward products) or [K,N]
// (C = A B_e, the input gradients).  Tiles are numbered row tile by row tile (T-row tiles counted
// over all experts, an expert's last one may be short), column tiles fastest.  The hardware hands
// workgroup b to XCD b % 8, each with an L2 of its own: XCD x takes the x-th contiguous eighth of
// the tile list, so that the workgroups it runs side by side share a few row tiles (every column
// tile of a row tile reads the same rows of A) and one or two experts' weights in its L2.
template <int T, bool B_KCONT>
__global__ __launch_bounds__(256) void f32_gemm_rows_kernel(F32Gemm p) {
  constexpr int LD = Shape<T>::LD, PER = Shape<T>::PER, NB = Shape<T>::NB;
  __shared__ __align__(16) float sA[TK * LD], sB[TK * LD];
  __shared__ int s_tile[3];
  const int n_col = (p.N + T - 1) / T;
  const long long total = (long long)(p.R / T + p.E) * n_col;  // (the grid's size)
  const long long chunk = (total + 7) / 8;
  const long long tile = (long long)(blockIdx.x % 8) * chunk + blockIdx.x / 8;
  if (blockIdx.x / 8 >= chunk || tile >= total) return;
  const int row_tile = (int)(tile / n_col), col_tile = (int)(tile % n_col);
  if (threadIdx.x == 0) {
    int seen = 0, found = -1, row0 = 0, row_end = 0;
    for (int e = 0; e < p.E; ++e) {
      const int b = p.offs[e], n = p.offs[e + 1] - b;
      if (n <= 0 || b < 0 || b + n > p.R) continue;  // (empty, or offsets no dispatch would produce)
      const int nt = (n + T - 1) / T;
      if (row_tile < seen + nt) {
        found = e;
        row0 = b + (row_tile - seen) * T;
        row_end = b + n;
        break;
      }
      seen += nt;
    }
    s_tile[0] = found;
    s_tile[1] = row0;
    s_tile[2] = row_end;
  }
  __syncthreads();
  const int e = s_tile[0], row0 = s_tile[1], row_end = s_tile[2];
  if (e < 0) return;  // (the grid is sized for the worst case: R/T + E row tiles)
  const int n0 = col_tile * T;
  const float* Be = p.B + (long long)e * p.N * p.K;
  const int wv = threadIdx.x >> 6, wm = wv >> 1, wn = wv & 1;
  f32x16 acc[NB][NB];
  clear<T>(acc);
  f32x4 ra[PER], rb[PER];
  auto fetch = [&](int k0) {
    load_kcont<T>(ra, p.A, p.K, row0, row_end, k0, p.K);
    if constexpr (B_KCONT) load_kcont<T>(rb, Be, p.K, n0, p.N, k0, p.K);
    else load_icont<T>(rb, Be, p.N, k0, p.K, n0, p.N);
  };
  fetch(0);
  for (int k0 = 0; k0 < p.K; k0 += TK) {
    stage_kcont<T>(sA, ra);
    if constexpr (B_KCONT) stage_kcont<T>(sB, rb);
    else stage_icont<T>(sB, rb);
    __syncthreads();
    if (k0 + TK < p.K) fetch(k0 + TK);
    mma_tile<T>(sA, sB, wm, wn, acc);
    __syncthreads();
  }
  store_tile<T>(p.C, p.N, row0, row_end, n0, p.N, wm, wn, acc, p.accumulate != 0);
}

// k-ragged: C_e[m, n] (+)= sum over the rows r of expert e of A[r, m] * B[r, n]  (the weight
// gradients).  A [R,M], B [R,N] row-major, C [E,M,N].  Tiles are numbered expert by expert and an
// XCD takes a contiguous eighth of them (as in the kernel above): the workgroups an XCD runs side
// by side then walk the rows of one or two experts together and find them in its L2.  An expert
// without rows gets zeros (or is left alone when accumulating).
template <int T>
__global__ __launch_bounds__(256) void f32_gemm_wgrad_kernel(F32Gemm p) {
  constexpr int LD = Shape<T>::LD, PER = Shape<T>::PER, NB = Shape<T>::NB;
  __shared__ __align__(16) float sA[TK * LD], sB[TK * LD];
  const int n_col = (p.N + T - 1) / T, n_row = (p.M + T - 1) / T;
  const long long total = (long long)p.E * n_row * n_col;
  const long long chunk = (total + 7) / 8;
  const long long tile = (long long)(blockIdx.x % 8) * chunk + blockIdx.x / 8;
  if (blockIdx.x / 8 >= chunk || tile >= total) return;
  const int e = (int)(tile / ((long long)n_row * n_col));
  const int in_e = (int)(tile % ((long long)n_row * n_col));
  const int n0 = (in_e % n_col) * T, m0 = (in_e / n_col) * T;
  int b = p.offs[e], end = p.offs[e + 1];
  if (b < 0 || end > p.R || end < b) b = end = 0;
  const int wv = threadIdx.x >> 6, wm = wv >> 1, wn = wv & 1;
  f32x16 acc[NB][NB];
  clear<T>(acc);
  f32x4 ra[PER], rb[PER];
  load_icont<T>(ra, p.A, p.M, b, end, m0, p.M);
  load_icont<T>(rb, p.B, p.N, b, end, n0, p.N);
  for (int k0 = b; k0 < end; k0 += TK) {
    stage_icont<T>(sA, ra);
    stage_icont<T>(sB, rb);
    __syncthreads();
    if (k0 + TK < end) {
      load_icont<T>(ra, p.A, p.M, k0 + TK, end, m0, p.M);
      load_icont<T>(rb, p.B, p.N, k0 + TK, end, n0, p.N);
    }
    mma_tile<T>(sA, sB, wm, wn, acc);
    __syncthreads();
  }
  if (end == b && p.accumulate) return;
  store_tile<T>(p.C + (long long)e * p.M * p.N, p.N, m0, p.M, n0, p.N, wm, wn, acc, p.accumulate != 0);
}

// The larger tile halves the operand traffic per flop; a launch takes it when it still gives
// every compute unit at least two tiles.
int f32_forced_tile = 0;
int f32_units[MOE_MAX_DEVICES];
int f32_compute_units() {
  const int dev = moe_current_device();
  if (f32_units[dev] <= 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    f32_units[dev] = n;
  }
  return f32_units[dev];
}
bool f32_large_tiles(int64_t tiles128) {
  if (f32_forced_tile) return f32_forced_tile == 128;
  return tiles128 >= 2 * (int64_t)f32_compute_units();
}

// ---- row movers and element-wise kernels (one workgroup per row, 16-byte accesses)

// xp[pos, :] = x[pos_to_row[pos] / k, :]   (mlp.py:104-131: repeat_interleave + the two sorts)
__global__ __launch_bounds__(256) void f32_gather_rows_kernel(const float* __restrict__ x,
                                                              const int32_t* __restrict__ pos_to_row, int T,
                                                              int H, int k, float* __restrict__ xp) {
  const long long pos = blockIdx.x;
  const int row = pos_to_row[pos];
  const int t = row / k;
  const bool ok = row >= 0 && t < T;
  for (int h = threadIdx.x * 4; h < H; h += 256 * 4) {
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (ok) v = *reinterpret_cast<const f32x4*>(x + (long long)t * H + h);
    *reinterpret_cast<f32x4*>(xp + pos * H + h) = v;
  }
}

// out[t, :] = sum_j gates[t*k+j] * y[row_to_pos[t*k+j], :], j ascending  (mlp.py:160-169);
// gates == nullptr: all ones (with k = 1 a pure un-permute)
__global__ __launch_bounds__(256) void f32_combine_fwd_kernel(const float* __restrict__ y,
                                                              const float* __restrict__ gates,
                                                              const int32_t* __restrict__ row_to_pos, int R,
                                                              int H, int k, float* __restrict__ out) {
  const long long t = blockIdx.x;
  for (int h = threadIdx.x * 4; h < H; h += 256 * 4) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const int pos = row_to_pos[t * k + j];
      if (pos < 0 || pos >= R) continue;
      const float g = gates ? gates[t * k + j] : 1.f;
      const f32x4 v = *reinterpret_cast<const f32x4*>(y + (long long)pos * H + h);
      acc += g * v;
    }
    *reinterpret_cast<f32x4*>(out + t * H + h) = acc;
  }
}

// Backward of the above: dyp[pos, :] = gate * dy[t, :], dgates[row] = <dy[t, :], y[pos, :]>
// (row = pos_to_row[pos], t = row / k).  The dot product is reduced in a fixed tree.
__global__ __launch_bounds__(256) void f32_combine_bwd_kernel(const float* __restrict__ dy,
                                                              const float* __restrict__ y,
                                                              const float* __restrict__ gates,
                                                              const int32_t* __restrict__ pos_to_row, int T,
                                                              int H, int k, float* __restrict__ dyp,
                                                              float* __restrict__ dgates) {
  __shared__ float part[4];
  const long long pos = blockIdx.x;
  const int row = pos_to_row[pos];
  const int t = row / k;
  const bool ok = row >= 0 && t < T;
  const float g = ok ? (gates ? gates[row] : 1.f) : 0.f;
  float dot = 0.f;
  for (int h = threadIdx.x * 4; h < H; h += 256 * 4) {
    f32x4 d = {0.f, 0.f, 0.f, 0.f};
    if (ok) d = *reinterpret_cast<const f32x4*>(dy + (long long)t * H + h);
    *reinterpret_cast<f32x4*>(dyp + pos * H + h) = g * d;
    if (dgates) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(y + pos * H + h);
      dot += d[0] * v[0] + d[1] * v[1] + d[2] * v[2] + d[3] * v[3];
    }
  }
  if (!dgates) return;  // (uniform: every thread leaves)
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o, MOE_WAVE);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = dot;
  __syncthreads();
  if (threadIdx.x == 0 && ok) dgates[row] = (part[0] + part[1]) + (part[2] + part[3]);
}

// dx[t, :] = sum_j dxp[row_to_pos[t*k+j], :], j ascending  (backward of the replication)
__global__ __launch_bounds__(256) void f32_permute_bwd_kernel(const float* __restrict__ dxp,
                                                              const int32_t* __restrict__ row_to_pos, int R,
                                                              int H, int k, float* __restrict__ dx) {
  const long long t = blockIdx.x;
  for (int h = threadIdx.x * 4; h < H; h += 256 * 4) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < k; ++j) {
      const int pos = row_to_pos[t * k + j];
      if (pos < 0 || pos >= R) continue;
      acc += *reinterpret_cast<const f32x4*>(dxp + (long long)pos * H + h);
    }
    *reinterpret_cast<f32x4*>(dx + t * H + h) = acc;
  }
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.f / (1.f + expf(-x)); }

// act = silu(g) * u   (mlp.py:156)
__global__ __launch_bounds__(256) void f32_swiglu_fwd_kernel(const float* __restrict__ g,
                                                             const float* __restrict__ u, long long n4,
                                                             float* __restrict__ act) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const f32x4 gv = reinterpret_cast<const f32x4*>(g)[i], uv = reinterpret_cast<const f32x4*>(u)[i];
  f32x4 a;
#pragma unroll
  for (int x = 0; x < 4; ++x) a[x] = gv[x] * sigmoid_f32(gv[x]) * uv[x];
  reinterpret_cast<f32x4*>(act)[i] = a;
}

// dg = dact * u * silu'(g), du = dact * silu(g);  silu'(g) = s * (1 + g * (1 - s)), s = sigmoid(g)
__global__ __launch_bounds__(256) void f32_swiglu_bwd_kernel(const float* __restrict__ dact,
                                                             const float* __restrict__ g,
                                                             const float* __restrict__ u, long long n4,
                                                             float* __restrict__ dg, float* __restrict__ du) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n4) return;
  const f32x4 dv = reinterpret_cast<const f32x4*>(dact)[i];
  const f32x4 gv = reinterpret_cast<const f32x4*>(g)[i], uv = reinterpret_cast<const f32x4*>(u)[i];
  f32x4 a, b;
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    const float s = sigmoid_f32(gv[x]);
    a[x] = dv[x] * uv[x] * (s * (1.f + gv[x] * (1.f - s)));
    b[x] = dv[x] * (gv[x] * s);
  }
  reinterpret_cast<f32x4*>(dg)[i] = a;
  reinterpret_cast<f32x4*>(du)[i] = b;
}

int check_rows(int64_t rows, int64_t width) {
  if (rows < 0 || width <= 0 || width % 4 != 0) return MOE_ERR_SHAPE;
  if (rows > (int64_t)1 << 30 || width > 65536) return MOE_ERR_LIMIT;
  return 0;
}

}  // namespace

extern "C" int moe_f32_gather_rows(const float* x, const int32_t* pos_to_row, int64_t T, int64_t R, int64_t H,
                                   int64_t k, float* xp, void* stream) {
  if (int rc = check_rows(R, H)) return rc;
  if (T < 0 || k <= 0) return MOE_ERR_SHAPE;
  if (T > (int64_t)1 << 30 || k > MOE_MAX_TOPK) return MOE_ERR_LIMIT;
  if (R == 0) return 0;
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(xp);
  if (!pos_to_row) return MOE_ERR_NULL;
  hipLaunchKernelGGL(f32_gather_rows_kernel, dim3((unsigned)R), dim3(256), 0, (hipStream_t)stream, x, pos_to_row,
                     (int)T, (int)H, (int)k, xp);
  return moe_launch_status();
}

extern "C" int moe_f32_combine_fwd(const float* y, const float* gates, const int32_t* row_to_pos, int64_t T,
                                   int64_t H, int64_t k, float* out, void* stream) {
  if (int rc = check_rows(T, H)) return rc;
  if (k <= 0) return MOE_ERR_SHAPE;
  if (k > MOE_MAX_TOPK || T * k > (int64_t)1 << 30) return MOE_ERR_LIMIT;
  if (T == 0) return 0;
  MOE_CHECK_PTR(y);
  MOE_CHECK_PTR(out);
  if (!row_to_pos) return MOE_ERR_NULL;
  hipLaunchKernelGGL(f32_combine_fwd_kernel, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream, y, gates,
                     row_to_pos, (int)(T * k), (int)H, (int)k, out);
  return moe_launch_status();
}

extern "C" int moe_f32_combine_bwd(const float* dy, const float* y, const float* gates,
                                   const int32_t* pos_to_row, int64_t T, int64_t R, int64_t H, int64_t k,
                                   float* dyp, float* dgates, void* stream) {
  if (int rc = check_rows(R, H)) return rc;
  if (T < 0 || k <= 0) return MOE_ERR_SHAPE;
  if (T > (int64_t)1 << 30 || k > MOE_MAX_TOPK) return MOE_ERR_LIMIT;
  if (R == 0) return 0;
  MOE_CHECK_PTR(dy);
  MOE_CHECK_PTR(dyp);
  if (!pos_to_row) return MOE_ERR_NULL;
  if (dgates) MOE_CHECK_PTR(y);
  hipLaunchKernelGGL(f32_combine_bwd_kernel, dim3((unsigned)R), dim3(256), 0, (hipStream_t)stream, dy, y, gates,
                     pos_to_row, (int)T, (int)H, (int)k, dyp, dgates);
  return moe_launch_status();
}

extern "C" int moe_f32_permute_bwd(const float* dxp, const int32_t* row_to_pos, int64_t T, int64_t H, int64_t k,
                                   float* dx, void* stream) {
  if (int rc = check_rows(T, H)) return rc;
  if (k <= 0) return MOE_ERR_SHAPE;
  if (k > MOE_MAX_TOPK || T * k > (int64_t)1 << 30) return MOE_ERR_LIMIT;
  if (T == 0) return 0;
  MOE_CHECK_PTR(dxp);
  MOE_CHECK_PTR(dx);
  if (!row_to_pos) return MOE_ERR_NULL;
  hipLaunchKernelGGL(f32_permute_bwd_kernel, dim3((unsigned)T), dim3(256), 0, (hipStream_t)stream, dxp, row_to_pos,
                     (int)(T * k), (int)H, (int)k, dx);
  return moe_launch_status();
}

extern "C" int moe_f32_swiglu_fwd(const float* g, const float* u, int64_t n, float* act, void* stream) {
  if (n < 0 || n % 4 != 0) return MOE_ERR_SHAPE;
  if (n == 0) return 0;
  if (n / 4 > (int64_t)0x7fffffff * 256) return MOE_ERR_LIMIT;
  MOE_CHECK_PTR(g);
  MOE_CHECK_PTR(u);
  MOE_CHECK_PTR(act);
  const long long n4 = n / 4;
  hipLaunchKernelGGL(f32_swiglu_fwd_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     g, u, n4, act);
  return moe_launch_status();
}

extern "C" int moe_f32_swiglu_bwd(const float* dact, const float* g, const float* u, int64_t n, float* dg,
                                  float* du, void* stream) {
  if (n < 0 || n % 4 != 0) return MOE_ERR_SHAPE;
  if (n == 0) return 0;
  if (n / 4 > (int64_t)0x7fffffff * 256) return MOE_ERR_LIMIT;
  MOE_CHECK_PTR(dact);
  MOE_CHECK_PTR(g);
  MOE_CHECK_PTR(u);
  MOE_CHECK_PTR(dg);
  MOE_CHECK_PTR(du);
  const long long n4 = n / 4;
  hipLaunchKernelGGL(f32_swiglu_bwd_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     dact, g, u, n4, dg, du);
  return moe_launch_status();
}

extern "C" int moe_f32_gemm_rows(const float* a, const float* b, const int32_t* offs, int64_t E, int64_t R,
                                 int64_t N, int64_t K, int b_k_contiguous, float* c, int accumulate,
                                 void* stream) {
  if (int rc = check_rows(R, N)) return rc;
  if (int rc = check_rows(R, K)) return rc;
  if (E <= 0) return MOE_ERR_SHAPE;
  if (E > 1024) return MOE_ERR_LIMIT;
  if (R == 0) return 0;
  MOE_CHECK_PTR(a);
  MOE_CHECK_PTR(b);
  MOE_CHECK_PTR(c);
  if (!offs) return MOE_ERR_NULL;
  F32Gemm p{a, b, c, offs, (int)E, (int)R, 0, (int)N, (int)K, accumulate};
  hipStream_t s = (hipStream_t)stream;
  // (one workgroup per tile slot, rounded up to whole eighths: see the kernel's tile numbering)
  auto blocks = [&](int64_t t) { return (unsigned)(((R / t + E) * ((N + t - 1) / t) + 7) / 8 * 8); };
  if ((R / 64 + E) * ((N + 63) / 64) + 8 > 0x7fffffffll) return MOE_ERR_LIMIT;
  if (f32_large_tiles((R / 128 + E) * ((N + 127) / 128))) {
    if (b_k_contiguous) hipLaunchKernelGGL((f32_gemm_rows_kernel<128, true>), dim3(blocks(128)), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((f32_gemm_rows_kernel<128, false>), dim3(blocks(128)), dim3(256), 0, s, p);
  } else {
    if (b_k_contiguous) hipLaunchKernelGGL((f32_gemm_rows_kernel<64, true>), dim3(blocks(64)), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((f32_gemm_rows_kernel<64, false>), dim3(blocks(64)), dim3(256), 0, s, p);
  }
  return moe_launch_status();
}

extern "C" int moe_f32_gemm_wgrad(const float* a, const float* b, const int32_t* offs, int64_t E, int64_t R,
                                  int64_t M, int64_t N, float* dw, int accumulate, void* stream) {
  if (int rc = check_rows(R, M)) return rc;
  if (int rc = check_rows(R, N)) return rc;
  if (E <= 0) return MOE_ERR_SHAPE;
  if (E > 1024) return MOE_ERR_LIMIT;
  MOE_CHECK_PTR(dw);
  if (!offs) return MOE_ERR_NULL;
  if (R > 0) {
    MOE_CHECK_PTR(a);
    MOE_CHECK_PTR(b);
  }
  F32Gemm p{a, b, dw, offs, (int)E, (int)R, (int)M, (int)N, 0, accumulate};
  auto blocks = [&](int64_t t) { return (unsigned)((E * ((M + t - 1) / t) * ((N + t - 1) / t) + 7) / 8 * 8); };
  if (E * ((M + 63) / 64) * ((N + 63) / 64) + 8 > 0x7fffffffll) return MOE_ERR_LIMIT;
  if (f32_large_tiles(E * ((M + 127) / 128) * ((N + 127) / 128)))
    hipLaunchKernelGGL(f32_gemm_wgrad_kernel<128>, dim3(blocks(128)), dim3(256), 0, (hipStream_t)stream, p);
  else
    hipLaunchKernelGGL(f32_gemm_wgrad_kernel<64>, dim3(blocks(64)), dim3(256), 0, (hipStream_t)stream, p);
  return moe_launch_status();
}

// Test hook: 0 lets every fp32 GEMM launch choose its tile (the default), 64 or 128 forces it.
// Process-wide and not synchronised: for tests, not for production callers.  Returns the previous
// setting.
extern "C" int moe_f32_gemm_force_tile(int t) {
  const int before = f32_forced_tile;
  if (t == 0 || t == 64 || t == 128) f32_forced_tile = t;
  return before;
}
