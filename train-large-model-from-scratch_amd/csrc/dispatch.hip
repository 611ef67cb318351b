// Dispatch / combine side of the MoE path for gfx950: per-expert histogram, prefix scan,
// stable permutation, row gather, weighted un-permute and their backward passes.  All of
// these are HBM-bound row movers; rows travel as 16-byte vectors (8 bf16).
//
// Stable counting sort in three launches:
//   1. every wavefront owns 256 consecutive routed rows and builds its own histogram in
//      LDS with LDS atomics (order-independent, hence deterministic);
//   2. one wavefront per expert turns the column of per-wave histograms into an exclusive
//      prefix (wave shuffles) and emits the expert's total count;
//   3. every wavefront re-reads its rows, finds the lanes that hold the same expert with
//      ballots, and gives row r the position offs[e] + rows-of-e-in-earlier-waves +
//      rows-of-e-earlier-in-this-wave -- i.e. the stable order -- writing both the
//      permutation and its inverse.
#include <mutex>

#include "common.h"

namespace {

constexpr int ROWS_PER_WAVE = 256;
constexpr int WAVES_PER_BLOCK = 4;

__device__ __forceinline__ int wave_incl_scan(int v) {
  const int lane = lane_id();
#pragma unroll
  for (int off = 1; off < MOE_WAVE; off <<= 1) {
    int o = __shfl_up(v, off, MOE_WAVE);
    if (lane >= off) v += o;
  }
  return v;
}

__device__ __forceinline__ int clamp_expert(int e, int E) { return e < 0 ? 0 : (e >= E ? E - 1 : e); }

// whist [NW][E] per-wave histograms; wbad [NW] per-wave counts of ids outside [0, E) (such a
// row is counted, and later placed, with the nearest valid expert so that every position of
// the permutation is still written; the count is how the caller learns of it).
__global__ __launch_bounds__(256) void hist_kernel(const int32_t* __restrict__ ids, int R, int E,
                                                  int NW, int32_t* __restrict__ whist,
                                                  int32_t* __restrict__ wbad) {
  extern __shared__ int cnt[];  // [WAVES_PER_BLOCK][E]
  const int lane = lane_id(), wv = threadIdx.x / MOE_WAVE;
  const int w = blockIdx.x * WAVES_PER_BLOCK + wv;
  int* mine = cnt + wv * E;
  for (int e = lane; e < E; e += MOE_WAVE) mine[e] = 0;
  __syncthreads();
  int bad = 0;
  if (w < NW) {
    const int base = w * ROWS_PER_WAVE;
#pragma unroll
    for (int it = 0; it < ROWS_PER_WAVE / MOE_WAVE; ++it) {
      const int r = base + it * MOE_WAVE + lane;
      if (r < R) {
        const int e = ids[r];
        bad += (e < 0 || e >= E) ? 1 : 0;
        atomicAdd(&mine[clamp_expert(e, E)], 1);
      }
    }
  }
  __syncthreads();
  if (w < NW) {
    for (int e = lane; e < E; e += MOE_WAVE) whist[(size_t)w * E + e] = mine[e];
#pragma unroll
    for (int off = MOE_WAVE / 2; off > 0; off >>= 1) bad += __shfl_xor(bad, off, MOE_WAVE);
    if (lane == 0) wbad[w] = bad;
  }
}

// One wave per expert: exclusive scan down the column whist[:, e]; counts[e] = total.
// Block E (one past the experts) adds up the per-wave counts of invalid ids into *bad_total
// (when the caller asked for it).
__global__ __launch_bounds__(64) void colscan_kernel(int32_t* __restrict__ whist, int NW, int E,
                                                    int32_t* __restrict__ counts,
                                                    const int32_t* __restrict__ wbad,
                                                    int32_t* __restrict__ bad_total) {
  const int e = blockIdx.x, lane = lane_id();
  if (e == E) {
    int sum = 0;
    for (int w = lane; w < NW; w += MOE_WAVE) sum += wbad[w];
#pragma unroll
    for (int off = MOE_WAVE / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, MOE_WAVE);
    if (lane == 0) *bad_total = sum;
    return;
  }
  int running = 0;
  for (int base = 0; base < NW; base += MOE_WAVE) {
    const int w = base + lane;
    const int v = w < NW ? whist[(size_t)w * E + e] : 0;
    const int incl = wave_incl_scan(v);
    if (w < NW) whist[(size_t)w * E + e] = running + incl - v;
    running += __shfl(incl, MOE_WAVE - 1, MOE_WAVE);
  }
  if (lane == 0) counts[e] = running;
}

__global__ __launch_bounds__(256) void positions_kernel(const int32_t* __restrict__ ids, int R,
                                                       int E, int NW,
                                                       const int32_t* __restrict__ whist,
                                                       const int32_t* __restrict__ counts,
                                                       int32_t* __restrict__ offs,
                                                       int32_t* __restrict__ pos_to_row,
                                                       int32_t* __restrict__ row_to_pos) {
  extern __shared__ int cnt[];  // [WAVES_PER_BLOCK][E] running write cursors
  const int lane = lane_id(), wv = threadIdx.x / MOE_WAVE;
  const int w = blockIdx.x * WAVES_PER_BLOCK + wv;
  int* cur = cnt + wv * E;
  const bool live = w < NW;
  // exclusive scan of counts over experts (every wave repeats it: E <= 512 values)
  int carry = 0;
  for (int b = 0; b < E; b += MOE_WAVE) {
    const int e = b + lane;
    const int c = e < E ? counts[e] : 0;
    const int incl = wave_incl_scan(c);
    if (e < E) {
      const int start = carry + incl - c;
      cur[e] = start + (live ? whist[(size_t)w * E + e] : 0);
      if (w == 0) offs[e] = start;
    }
    carry += __shfl(incl, MOE_WAVE - 1, MOE_WAVE);
  }
  if (w == 0 && lane == 0) offs[E] = carry;
  __syncthreads();
  if (!live) return;
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  const int base = w * ROWS_PER_WAVE;
  for (int it = 0; it < ROWS_PER_WAVE / MOE_WAVE; ++it) {
    const int r = base + it * MOE_WAVE + lane;
    const bool valid = r < R;
    const int e = valid ? clamp_expert(ids[r], E) : 0;
    unsigned long long mask = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
      const bool bit = (e >> b) & 1;
      const unsigned long long bal = __ballot(valid && bit);
      mask &= bit ? bal : ~bal;
    }
    const unsigned long long lt = (1ull << lane) - 1ull;
    const int rank = __popcll(mask & lt);
    int old = 0;
    if (valid) old = cur[e];
    __builtin_amdgcn_wave_barrier();
    if (valid && rank == 0) cur[e] = old + __popcll(mask);
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      const int pos = old + rank;
      pos_to_row[pos] = r;
      row_to_pos[r] = pos;
    }
  }
}

// The three kernels above as one, for inputs small enough that a single workgroup's LDS holds
// every chunk's histogram (SMALL_MAX_CHUNKS * E ints): 16 waves take the 256-row chunks in turn,
// the histograms, their column scans and the running cursors never leave LDS, and two launches
// (and their gaps) are saved where the whole layer step is a few tens of microseconds.  Same
// chunking, same stable ranks: the results are the same bits as the three-kernel path.
constexpr int SMALL_WAVES = 16;
constexpr int SMALL_MAX_CHUNKS = 16;         // one chunk per wave, R <= 4096: at 64 chunks (16384 rows) the one
                                             // workgroup takes 19 us where the three kernels take 11
constexpr int SMALL_MAX_WORDS = 12 * 1024;   // chunks * E ints of LDS (48 KB)

__global__ __launch_bounds__(SMALL_WAVES* MOE_WAVE) void dispatch_small_kernel(
    const int32_t* __restrict__ ids, int R, int E, int NW, int32_t* __restrict__ counts,
    int32_t* __restrict__ offs, int32_t* __restrict__ pos_to_row, int32_t* __restrict__ row_to_pos,
    int32_t* __restrict__ bad_total) {
  extern __shared__ int sm[];  // [NW][E] chunk histograms, later write cursors; [E] starts; [1] bad
  int* whist = sm;
  int* starts = sm + NW * E;
  int* bad_sum = starts + E;
  const int lane = lane_id(), wv = threadIdx.x / MOE_WAVE;
  for (int i = threadIdx.x; i < NW * E + E + 1; i += blockDim.x) sm[i] = 0;
  __syncthreads();
  // per-chunk histograms
  int bad = 0;
  for (int w = wv; w < NW; w += SMALL_WAVES) {
    const int base = w * ROWS_PER_WAVE;
#pragma unroll
    for (int it = 0; it < ROWS_PER_WAVE / MOE_WAVE; ++it) {
      const int r = base + it * MOE_WAVE + lane;
      if (r < R) {
        const int e = ids[r];
        bad += (e < 0 || e >= E) ? 1 : 0;
        atomicAdd(&whist[w * E + clamp_expert(e, E)], 1);
      }
    }
  }
#pragma unroll
  for (int off = MOE_WAVE / 2; off > 0; off >>= 1) bad += __shfl_xor(bad, off, MOE_WAVE);
  if (lane == 0 && bad) atomicAdd(bad_sum, bad);
  __syncthreads();
  // exclusive scan down every expert's column of chunk counts (NW <= 64 lanes: one pass of a wave)
  for (int e = wv; e < E; e += SMALL_WAVES) {
    const int v = lane < NW ? whist[lane * E + e] : 0;
    const int incl = wave_incl_scan(v);
    if (lane < NW) whist[lane * E + e] = incl - v;
    if (lane == MOE_WAVE - 1) {
      starts[e] = incl;  // the expert's count, for the moment
      counts[e] = incl;
    }
  }
  __syncthreads();
  // exclusive scan of the counts over the experts (wave 0), then the cursors of every chunk
  if (wv == 0) {
    int carry = 0;
    for (int b = 0; b < E; b += MOE_WAVE) {
      const int e = b + lane;
      const int c = e < E ? starts[e] : 0;
      const int incl = wave_incl_scan(c);
      if (e < E) {
        const int st = carry + incl - c;
        starts[e] = st;
        offs[e] = st;
      }
      carry += __shfl(incl, MOE_WAVE - 1, MOE_WAVE);  // (every lane takes part: not inside the branch)
    }
    if (lane == 0) {
      offs[E] = carry;
      if (bad_total) *bad_total = *bad_sum;
    }
  }
  __syncthreads();
  int nbits = 0;
  while ((1 << nbits) < E) ++nbits;
  for (int w = wv; w < NW; w += SMALL_WAVES) {
    int* cur = whist + w * E;
    for (int e = lane; e < E; e += MOE_WAVE) cur[e] += starts[e];
    __builtin_amdgcn_wave_barrier();
    const int base = w * ROWS_PER_WAVE;
    for (int it = 0; it < ROWS_PER_WAVE / MOE_WAVE; ++it) {
      const int r = base + it * MOE_WAVE + lane;
      const bool valid = r < R;
      const int e = valid ? clamp_expert(ids[r], E) : 0;
      unsigned long long mask = __ballot(valid);
      for (int b = 0; b < nbits; ++b) {
        const bool bit = (e >> b) & 1;
        const unsigned long long bal = __ballot(valid && bit);
        mask &= bit ? bal : ~bal;
      }
      const unsigned long long lt = (1ull << lane) - 1ull;
      const int rank = __popcll(mask & lt);
      int old = 0;
      if (valid) old = cur[e];
      __builtin_amdgcn_wave_barrier();
      if (valid && rank == 0) cur[e] = old + __popcll(mask);
      __builtin_amdgcn_wave_barrier();
      if (valid) {
        const int pos = old + rank;
        pos_to_row[pos] = r;
        row_to_pos[r] = pos;
      }
    }
  }
}

// ---- row movers ---------------------------------------------------------------------------

constexpr int ROWS_PER_BLOCK = 4;
constexpr int64_t MAX_ROW_ELEMS = 65536;  // widest row the movers take (H and I <= 65536 throughout)

// xp[pos,:] = bf16(x[pos_to_row[pos]/k,:])
template <typename XT>
__global__ __launch_bounds__(256) void permute_fwd_kernel(const XT* __restrict__ x,
                                                         const int32_t* __restrict__ pos_to_row,
                                                         int R, int H8, int k,
                                                         uint16_t* __restrict__ xp) {
  const int H = H8 * 8;
  const bool once = (k == 1);  // every source row is read exactly once: streaming loads
  if constexpr (sizeof(XT) == 2) {
    // a pure row permutation of rows of up to 4096 elements: all of the block's loads are
    // requested before the first store, so that eight 16-byte loads per thread are in flight
    // instead of two
    if (once && H8 <= 512) {
      for (long long blk = blockIdx.x; blk * ROWS_PER_BLOCK < R; blk += gridDim.x) {
        const int row0 = (int)(blk * ROWS_PER_BLOCK);
        u32x4 v[ROWS_PER_BLOCK][2];
#pragma unroll
        for (int rr = 0; rr < ROWS_PER_BLOCK; ++rr) {
          const int pos = row0 + rr;
          const int t = pos < R ? pos_to_row[pos] : 0;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int col = (threadIdx.x + j * 256) * 8;
            if (pos < R && col < H)
              v[rr][j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + (size_t)t * H + col));
          }
        }
#pragma unroll
        for (int rr = 0; rr < ROWS_PER_BLOCK; ++rr) {
          const int pos = row0 + rr;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int col = (threadIdx.x + j * 256) * 8;
            if (pos < R && col < H) store_bits_nt(xp + (size_t)pos * H + col, v[rr][j]);
          }
        }
      }
      return;
    }
  }
  for (long long blk = blockIdx.x; blk * ROWS_PER_BLOCK < R; blk += gridDim.x) {
    const int row0 = (int)(blk * ROWS_PER_BLOCK);
#pragma unroll
    for (int rr = 0; rr < ROWS_PER_BLOCK; ++rr) {
      const int pos = row0 + rr;
      if (pos >= R) break;
      const int t = once ? pos_to_row[pos] : pos_to_row[pos] / k;
      const XT* src = x + (size_t)t * H;
      uint16_t* dst = xp + (size_t)pos * H;
      for (int col = threadIdx.x * 8; col < H; col += 256 * 8) {
        if constexpr (sizeof(XT) == 2) {  // bf16 -> bf16: move the bits
          const u32x4 bits = once ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + col))
                                  : *reinterpret_cast<const u32x4*>(src + col);
          store_bits_nt(dst + col, bits);
        } else {
          store8_nt(dst + col, load8(src + col));
        }
      }
    }
  }
}

// The same rows written token by token: x[t,:] is read once and stored to its k places
// xp[row_to_pos[t*k+j],:].  One read feeds k independent stores, and the source is walked in
// order instead of gathered.
template <typename XT>
__global__ __launch_bounds__(256) void permute_fwd_scatter_kernel(const XT* __restrict__ x,
                                                                 const int32_t* __restrict__ row_to_pos,
                                                                 int T, int H8, int k,
                                                                 uint16_t* __restrict__ xp) {
  const int H = H8 * 8;
  for (long long blk = blockIdx.x; blk * ROWS_PER_BLOCK < T; blk += gridDim.x) {
    const int row0 = (int)(blk * ROWS_PER_BLOCK);
    for (int c = threadIdx.x; c < ROWS_PER_BLOCK * H8; c += blockDim.x) {
      const int t = row0 + c / H8, col = (c % H8) * 8;
      if (t >= T) continue;
      u32x4 bits;
      if constexpr (sizeof(XT) == 2) {
        bits = *reinterpret_cast<const u32x4*>(x + (size_t)t * H + col);
      } else {
        const Row8 v = load8(x + (size_t)t * H + col);
#pragma unroll
        for (int i = 0; i < 4; ++i) bits[i] = pack_bf16x2(v.v[2 * i], v.v[2 * i + 1]);
      }
      for (int j = 0; j < k; ++j) {
        const int pos = row_to_pos[(size_t)t * k + j];
        store_bits_nt(xp + (size_t)pos * H + col, bits);
      }
    }
  }
}

// out[t,:] = sum_j gates[t*k+j] * y[row_to_pos[t*k+j],:]  (+ addend[t,:]); fp32, slot order.
template <typename OT, typename AT>
__global__ __launch_bounds__(256) void combine_fwd_kernel(const uint16_t* __restrict__ y,
                                                         const float* __restrict__ gates,
                                                         const int32_t* __restrict__ row_to_pos,
                                                         const AT* __restrict__ addend, int T,
                                                         int H8, int k, OT* __restrict__ out) {
  const int H = H8 * 8;
  for (long long blk = blockIdx.x; blk * ROWS_PER_BLOCK < T; blk += gridDim.x) {
    const int row0 = (int)(blk * ROWS_PER_BLOCK);
    for (int c = threadIdx.x; c < ROWS_PER_BLOCK * H8; c += blockDim.x) {
      const int t = row0 + c / H8, col = (c % H8) * 8;
      if (t >= T) continue;
      Row8 acc;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc.v[i] = 0.f;
      int j = 0;
      for (; j + 8 <= k; j += 8) {  // eight rows in flight; summed in slot order all the same
        int pos[8];
        float gt[8];
        Row8 v[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          pos[q] = row_to_pos[(size_t)t * k + j + q];
          gt[q] = gates ? gates[(size_t)t * k + j + q] : 1.f;
        }
#pragma unroll
        for (int q = 0; q < 8; ++q) v[q] = load8_nt(y + (size_t)pos[q] * H + col);
#pragma unroll
        for (int q = 0; q < 8; ++q)
#pragma unroll
          for (int i = 0; i < 8; ++i) acc.v[i] += gt[q] * v[q].v[i];
      }
      for (; j + 4 <= k; j += 4) {  // four rows in flight; summed in slot order all the same
        int pos[4];
        float gt[4];
        Row8 v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          pos[q] = row_to_pos[(size_t)t * k + j + q];
          gt[q] = gates ? gates[(size_t)t * k + j + q] : 1.f;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = load8_nt(y + (size_t)pos[q] * H + col);
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int i = 0; i < 8; ++i) acc.v[i] += gt[q] * v[q].v[i];
      }
      for (; j < k; ++j) {
        const int pos = row_to_pos[(size_t)t * k + j];
        const float gt = gates ? gates[(size_t)t * k + j] : 1.f;
        const Row8 v = load8_nt(y + (size_t)pos * H + col);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc.v[i] += gt * v.v[i];
      }
      if (addend) {
        const Row8 a = load8(addend + (size_t)t * H + col);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc.v[i] += a.v[i];
      }
      store8(out + (size_t)t * H + col, acc);
    }
  }
}

// One wave per expert-ordered row: dyp[pos,:] = bf16(gate*dy[t,:]); dgates[r] = <dy[t], y[pos]>.
template <typename DT>
__global__ __launch_bounds__(256) void combine_bwd_kernel(const DT* __restrict__ dy,
                                                         const uint16_t* __restrict__ y,
                                                         const float* __restrict__ gates,
                                                         const int32_t* __restrict__ pos_to_row,
                                                         int R, int H8, int k,
                                                         uint16_t* __restrict__ dyp,
                                                         float* __restrict__ dgates) {
  const int H = H8 * 8, lane = lane_id();
  const int wpb = blockDim.x / MOE_WAVE;
  for (long long pos = (long long)blockIdx.x * wpb + threadIdx.x / MOE_WAVE; pos < R;
       pos += (long long)gridDim.x * wpb) {
    const int r = pos_to_row[pos];
    const int t = r / k;
    const float gt = gates ? gates[r] : 1.f;
    if constexpr (sizeof(DT) == 2) {
      // the scaled copy alone, rows of up to 4096 elements: the row's loads are all requested
      // before its first store (eight in flight per lane instead of one)
      if (!y && H8 <= 8 * MOE_WAVE) {
        u32x4 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int c = lane + j * MOE_WAVE;
          if (c < H8) {
            const u32x4* src = reinterpret_cast<const u32x4*>(dy + (size_t)t * H + c * 8);
            v[j] = (k == 1) ? __builtin_nontemporal_load(src) : *src;
          }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int c = lane + j * MOE_WAVE;
          if (c < H8) {
            Row8 d = row8_from_bits(v[j]);
#pragma unroll
            for (int i = 0; i < 8; ++i) d.v[i] *= gt;
            store8_nt(dyp + (size_t)pos * H + c * 8, d);
          }
        }
        continue;
      }
    }
    float dot = 0.f;
    for (int c = lane; c < H8; c += MOE_WAVE) {
      Row8 d;
      if constexpr (sizeof(DT) == 2) {  // k == 1: every row of dy is read exactly once
        d = (k == 1) ? load8_nt(dy + (size_t)t * H + c * 8) : load8(dy + (size_t)t * H + c * 8);
      } else {
        d = load8(dy + (size_t)t * H + c * 8);
      }
      if (y) {
        const Row8 yv = load8_nt(y + (size_t)pos * H + c * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) dot += d.v[i] * yv.v[i];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) d.v[i] *= gt;
      store8_nt(dyp + (size_t)pos * H + c * 8, d);
    }
    if (dgates) {
#pragma unroll
      for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, MOE_WAVE);
      if (lane == 0) dgates[r] = dot;
    }
  }
}

// The same, one wave per token: dy[t,:] is read once into registers (NV 16-byte groups per
// lane, H8 <= 64*NV) and serves the token's k routed rows.  Same per-lane summation order as
// the kernel above, hence the same bits.
template <typename DT, int NV>
__global__ __launch_bounds__(256) void combine_bwd_token_kernel(
    const DT* __restrict__ dy, const uint16_t* __restrict__ y, const float* __restrict__ gates,
    const int32_t* __restrict__ row_to_pos, int T, int H8, int k, uint16_t* __restrict__ dyp,
    float* __restrict__ dgates) {
  const int H = H8 * 8, lane = lane_id();
  const int wpb = blockDim.x / MOE_WAVE;
  for (long long t = (long long)blockIdx.x * wpb + threadIdx.x / MOE_WAVE; t < T;
       t += (long long)gridDim.x * wpb) {
    Row8 d[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int c = lane + i * MOE_WAVE;
      if (c < H8) d[i] = load8(dy + (size_t)t * H + c * 8);
    }
    for (int j = 0; j < k; ++j) {
      const long long r = t * k + j;
      const int pos = row_to_pos[r];
      const float gt = gates ? gates[r] : 1.f;
      float dot = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int c = lane + i * MOE_WAVE;
        if (c < H8) {
          Row8 o;
          if (y) {
            const Row8 yv = load8_nt(y + (size_t)pos * H + c * 8);
#pragma unroll
            for (int q = 0; q < 8; ++q) dot += d[i].v[q] * yv.v[q];
          }
#pragma unroll
          for (int q = 0; q < 8; ++q) o.v[q] = d[i].v[q] * gt;
          store8_nt(dyp + (size_t)pos * H + c * 8, o);
        }
      }
      if (dgates) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, MOE_WAVE);
        if (lane == 0) dgates[r] = dot;
      }
    }
  }
}

__global__ __launch_bounds__(256) void cast_kernel(const float* __restrict__ src,
                                                  uint16_t* __restrict__ dst, long long n8,
                                                  long long n) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (long long)gridDim.x * blockDim.x)
    store8(dst + i * 8, load8(src + i * 8));
  if (blockIdx.x == 0 && threadIdx.x < (n - n8 * 8))
    dst[n8 * 8 + threadIdx.x] = f32_to_bf16(src[n8 * 8 + threadIdx.x]);
}

inline unsigned mover_grid(int64_t rows, int per_block) {
  int64_t b = (rows + per_block - 1) / per_block;
  const int64_t cap = 256 * 16;  // 16 resident 256-thread blocks per CU is plenty for a copy
  return (unsigned)(b < 1 ? 1 : (b > cap ? cap : b));
}

}  // namespace

extern "C" int moe_abi_version(void) { return 101; }

extern "C" int64_t moe_dispatch_workspace_bytes(int64_t R, int64_t E) {
  if (R < 0 || E <= 0) return 0;
  const int64_t nw = (R + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
  return (nw > 0 ? nw : 1) * (E + 1) * (int64_t)sizeof(int32_t);  // [nw][E] histograms + [nw] invalid-id counts
}

namespace {

int histogram_scan_impl(const int32_t* ids, int64_t R, int64_t E, int32_t* counts, int32_t* offs,
                        int32_t* pos_to_row, int32_t* row_to_pos, int32_t* bad_ids, void* scratch,
                        hipStream_t s) {
  const int NW = (int)((R + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE);
  if (NW > 0 && NW <= SMALL_MAX_CHUNKS && (int64_t)NW * E <= SMALL_MAX_WORDS) {
    const size_t lds_small = ((size_t)NW * E + E + 1) * sizeof(int);
    hipLaunchKernelGGL(dispatch_small_kernel, dim3(1), dim3(SMALL_WAVES * MOE_WAVE), lds_small, s, ids, (int)R,
                       (int)E, NW, counts, offs, pos_to_row, row_to_pos, bad_ids);
    return moe_launch_status();
  }
  const int nblk = NW > 0 ? (NW + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK : 1;
  const size_t lds = (size_t)WAVES_PER_BLOCK * E * sizeof(int);
  int32_t* whist = (int32_t*)scratch;
  int32_t* wbad = whist + (size_t)(NW > 0 ? NW : 1) * E;
  if (NW > 0) {
    hipLaunchKernelGGL(hist_kernel, dim3(nblk), dim3(256), lds, s, ids, (int)R, (int)E, NW, whist, wbad);
  }
  hipLaunchKernelGGL(colscan_kernel, dim3((unsigned)E + (bad_ids ? 1u : 0u)), dim3(64), 0, s, whist, NW,
                     (int)E, counts, wbad, bad_ids);
  hipLaunchKernelGGL(positions_kernel, dim3(nblk), dim3(256), lds, s, ids, (int)R, (int)E, NW,
                     whist, counts, offs, pos_to_row, row_to_pos);
  return moe_launch_status();
}

int histogram_scan_args(const int32_t* ids, int64_t R, int64_t E, const int32_t* counts,
                        const int32_t* offs, const int32_t* pos_to_row, const int32_t* row_to_pos) {
  if (!counts || !offs) return MOE_ERR_NULL;
  if (R > 0 && (!ids || !pos_to_row || !row_to_pos)) return MOE_ERR_NULL;
  if (R < 0 || E <= 0) return MOE_ERR_SHAPE;
  if (E > MOE_MAX_EXPERTS || R > (int64_t)1 << 30) return MOE_ERR_LIMIT;
  return 0;
}

}  // namespace

extern "C" int moe_histogram_scan_checked(const int32_t* ids, int64_t R, int64_t E, int32_t* counts,
                                          int32_t* offs, int32_t* pos_to_row, int32_t* row_to_pos,
                                          int32_t* bad_ids, void* workspace, int64_t workspace_bytes,
                                          void* stream) {
  if (int rc = histogram_scan_args(ids, R, E, counts, offs, pos_to_row, row_to_pos)) return rc;
  if (!workspace) return MOE_ERR_NULL;
  if (workspace_bytes < moe_dispatch_workspace_bytes(R, E)) return MOE_ERR_WORKSPACE;
  return histogram_scan_impl(ids, R, E, counts, offs, pos_to_row, row_to_pos, bad_ids, workspace,
                             (hipStream_t)stream);
}

extern "C" int moe_histogram_scan(const int32_t* ids, int64_t R, int64_t E, int32_t* counts,
                                  int32_t* offs, int32_t* pos_to_row, int32_t* row_to_pos,
                                  void* workspace, int64_t workspace_bytes, void* stream) {
  return moe_histogram_scan_checked(ids, R, E, counts, offs, pos_to_row, row_to_pos, nullptr, workspace,
                                    workspace_bytes, stream);
}

// ---- the dispatch entry that allocates nothing -----------------------------------------------
// The per-wave histograms live in a fixed array in device memory that is part of the loaded
// code object: every GPU the library runs on holds its own copy at its own address until the
// process ends.  In host code the array's name is only a handle for the runtime; the address
// kernels can use is asked for once per device and kept.
#define MOE_STATIC_SCRATCH_BYTES (4 << 20)
static __device__ __align__(256) unsigned char scratch[MOE_STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = MOE_MAX_DEVICES;
void* scratch_of_device[MAX_DEVICES];  // device address of `scratch` on each GPU, 0 = not asked yet
std::mutex scratch_mutex;

// Device address of `scratch` on the current device (no allocation: a symbol lookup).
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= MAX_DEVICES) return MOE_ERR_LIMIT;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_of_device[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (!ptr) return MOE_ERR_NULL;
    scratch_of_device[dev] = ptr;
  }
  *out = scratch_of_device[dev];
  return 0;
}

}  // namespace

// Also the set-up call: it looks up the array's address on the current device, so that a caller
// who asks for the size before capturing a graph (or before entering a region that must not
// touch the runtime's symbol tables) leaves nothing for the first moe_histogram_scan_static to do.
extern "C" int64_t moe_static_scratch_bytes(void) {
  void* ptr = nullptr;
  (void)static_scratch(&ptr);
  return MOE_STATIC_SCRATCH_BYTES;
}

extern "C" int64_t moe_static_scratch_max_rows(int64_t E) {
  if (E <= 0 || E > MOE_MAX_EXPERTS) return 0;
  // largest R with moe_dispatch_workspace_bytes(R, E) <= the array: one (E + 1)-word histogram per
  // wave's chunk of rows
  const int64_t waves = MOE_STATIC_SCRATCH_BYTES / ((E + 1) * (int64_t)sizeof(int32_t));
  const int64_t rows = waves * ROWS_PER_WAVE;
  return rows < ((int64_t)1 << 30) ? rows : ((int64_t)1 << 30);
}

extern "C" int moe_histogram_scan_static(const int32_t* ids, int64_t R, int64_t E, int32_t* counts,
                                         int32_t* offs, int32_t* pos_to_row, int32_t* row_to_pos,
                                         int32_t* bad_ids, void* stream) {
  if (int rc = histogram_scan_args(ids, R, E, counts, offs, pos_to_row, row_to_pos)) return rc;
  if (moe_dispatch_workspace_bytes(R, E) > MOE_STATIC_SCRATCH_BYTES) return MOE_ERR_WORKSPACE;
  void* ptr = nullptr;
  if (int rc = static_scratch(&ptr)) return rc;
  // every word of the scratch that is read was written by this call's first kernel, so what
  // an earlier call left behind needs no clearing
  return histogram_scan_impl(ids, R, E, counts, offs, pos_to_row, row_to_pos, bad_ids, ptr,
                             (hipStream_t)stream);
}

extern "C" int moe_permute_fwd(const void* x, int x_dtype, const int32_t* pos_to_row, int64_t R,
                               int64_t H, int64_t k, uint16_t* xp, void* stream) {
  if (R == 0) return 0;
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(xp);
  if (!pos_to_row) return MOE_ERR_NULL;
  if (R < 0 || H <= 0 || k <= 0 || (H % 8) != 0) return MOE_ERR_SHAPE;
  if (R > (int64_t)1 << 30 || H > MAX_ROW_ELEMS || k > MOE_MAX_TOPK) return MOE_ERR_LIMIT;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(mover_grid(R, ROWS_PER_BLOCK)), block(256);
  if (x_dtype == MOE_DT_BF16)
    hipLaunchKernelGGL(permute_fwd_kernel<uint16_t>, grid, block, 0, s, (const uint16_t*)x,
                       pos_to_row, (int)R, (int)(H / 8), (int)k, xp);
  else if (x_dtype == MOE_DT_F32)
    hipLaunchKernelGGL(permute_fwd_kernel<float>, grid, block, 0, s, (const float*)x, pos_to_row,
                       (int)R, (int)(H / 8), (int)k, xp);
  else
    return MOE_ERR_DTYPE;
  return moe_launch_status();
}

extern "C" int moe_permute_fwd_scatter(const void* x, int x_dtype, const int32_t* row_to_pos,
                                       int64_t T, int64_t H, int64_t k, uint16_t* xp, void* stream) {
  if (T == 0) return 0;
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(xp);
  if (!row_to_pos) return MOE_ERR_NULL;
  if (T < 0 || H <= 0 || k <= 0 || (H % 8) != 0) return MOE_ERR_SHAPE;
  if (k > MOE_MAX_TOPK || T > (int64_t)1 << 30 || T * k > (int64_t)1 << 30 || H > MAX_ROW_ELEMS) return MOE_ERR_LIMIT;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(mover_grid(T, ROWS_PER_BLOCK)), block(256);
  if (x_dtype == MOE_DT_BF16)
    hipLaunchKernelGGL(permute_fwd_scatter_kernel<uint16_t>, grid, block, 0, s, (const uint16_t*)x,
                       row_to_pos, (int)T, (int)(H / 8), (int)k, xp);
  else if (x_dtype == MOE_DT_F32)
    hipLaunchKernelGGL(permute_fwd_scatter_kernel<float>, grid, block, 0, s, (const float*)x,
                       row_to_pos, (int)T, (int)(H / 8), (int)k, xp);
  else
    return MOE_ERR_DTYPE;
  return moe_launch_status();
}

static int combine_like(const uint16_t* y, const float* gates, const int32_t* row_to_pos,
                        const void* addend, int64_t T, int64_t H, int64_t k, void* out,
                        int out_dtype, void* stream, int addend_dtype = -1) {
  if (addend_dtype < 0) addend_dtype = out_dtype;
  if (T == 0) return 0;
  MOE_CHECK_PTR(y);
  MOE_CHECK_PTR(out);
  if (addend && !aligned16(addend)) return MOE_ERR_ALIGN;
  if (!row_to_pos) return MOE_ERR_NULL;
  if (T < 0 || H <= 0 || k <= 0 || (H % 8) != 0) return MOE_ERR_SHAPE;
  if (k > MOE_MAX_TOPK || T > (int64_t)1 << 30 || T * k > (int64_t)1 << 30 || H > MAX_ROW_ELEMS) return MOE_ERR_LIMIT;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(mover_grid(T, ROWS_PER_BLOCK)), block(256);
  if (out_dtype == MOE_DT_BF16 && addend_dtype == MOE_DT_BF16)
    hipLaunchKernelGGL((combine_fwd_kernel<uint16_t, uint16_t>), grid, block, 0, s, y, gates, row_to_pos,
                       (const uint16_t*)addend, (int)T, (int)(H / 8), (int)k, (uint16_t*)out);
  else if (out_dtype == MOE_DT_F32 && addend_dtype == MOE_DT_F32)
    hipLaunchKernelGGL((combine_fwd_kernel<float, float>), grid, block, 0, s, y, gates, row_to_pos,
                       (const float*)addend, (int)T, (int)(H / 8), (int)k, (float*)out);
  else if (out_dtype == MOE_DT_F32 && addend_dtype == MOE_DT_BF16)
    hipLaunchKernelGGL((combine_fwd_kernel<float, uint16_t>), grid, block, 0, s, y, gates, row_to_pos,
                       (const uint16_t*)addend, (int)T, (int)(H / 8), (int)k, (float*)out);
  else
    return MOE_ERR_DTYPE;
  return moe_launch_status();
}

extern "C" int moe_combine_fwd(const uint16_t* y, const float* gates, const int32_t* row_to_pos,
                               int64_t T, int64_t H, int64_t k, void* out, int out_dtype,
                               void* stream) {
  return combine_like(y, gates, row_to_pos, nullptr, T, H, k, out, out_dtype, stream);
}

extern "C" int moe_combine_fwd_residual(const uint16_t* y, const float* gates,
                                        const int32_t* row_to_pos, const void* residual,
                                        int64_t T, int64_t H, int64_t k, void* out, int out_dtype,
                                        void* stream) {
  if (T > 0 && !residual) return MOE_ERR_NULL;
  return combine_like(y, gates, row_to_pos, residual, T, H, k, out, out_dtype, stream);
}

extern "C" int moe_permute_bwd(const uint16_t* dxp, const int32_t* row_to_pos, const void* addend,
                               int64_t T, int64_t H, int64_t k, void* dx, int dx_dtype,
                               void* stream) {
  return combine_like(dxp, nullptr, row_to_pos, addend, T, H, k, dx, dx_dtype, stream);
}

extern "C" int moe_permute_bwd_addend(const uint16_t* dxp, const int32_t* row_to_pos,
                                      const void* addend, int addend_dtype, int64_t T, int64_t H,
                                      int64_t k, void* dx, int dx_dtype, void* stream) {
  if (T > 0 && !addend) return MOE_ERR_NULL;
  return combine_like(dxp, nullptr, row_to_pos, addend, T, H, k, dx, dx_dtype, stream, addend_dtype);
}

extern "C" int moe_combine_bwd(const void* dy, int dy_dtype, const uint16_t* y, const float* gates,
                               const int32_t* pos_to_row, int64_t R, int64_t H, int64_t k,
                               uint16_t* dyp, float* dgates, void* stream) {
  if (R == 0) return 0;
  MOE_CHECK_PTR(dy);
  MOE_CHECK_PTR(dyp);
  if (y && !aligned16(y)) return MOE_ERR_ALIGN;
  if (!pos_to_row) return MOE_ERR_NULL;
  if ((dgates != nullptr) != (y != nullptr)) return MOE_ERR_NULL;
  if (R < 0 || H <= 0 || k <= 0 || (H % 8) != 0) return MOE_ERR_SHAPE;
  if (R > (int64_t)1 << 30 || H > MAX_ROW_ELEMS || k > MOE_MAX_TOPK) return MOE_ERR_LIMIT;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(mover_grid(R, 4)), block(256);
  if (dy_dtype == MOE_DT_BF16)
    hipLaunchKernelGGL(combine_bwd_kernel<uint16_t>, grid, block, 0, s, (const uint16_t*)dy, y,
                       gates, pos_to_row, (int)R, (int)(H / 8), (int)k, dyp, dgates);
  else if (dy_dtype == MOE_DT_F32)
    hipLaunchKernelGGL(combine_bwd_kernel<float>, grid, block, 0, s, (const float*)dy, y, gates,
                       pos_to_row, (int)R, (int)(H / 8), (int)k, dyp, dgates);
  else
    return MOE_ERR_DTYPE;
  return moe_launch_status();
}

template <typename DT>
static int launch_combine_bwd_token(const void* dy, const uint16_t* y, const float* gates,
                                    const int32_t* row_to_pos, int64_t T, int64_t H, int64_t k,
                                    uint16_t* dyp, float* dgates, hipStream_t s) {
  const dim3 grid(mover_grid(T, 4)), block(256);
  const int64_t nv = (H / 8 + MOE_WAVE - 1) / MOE_WAVE;
#define MOE_CBT(NV)                                                                               \
  hipLaunchKernelGGL((combine_bwd_token_kernel<DT, NV>), grid, block, 0, s, (const DT*)dy, y, gates, \
                     row_to_pos, (int)T, (int)(H / 8), (int)k, dyp, dgates)
  if (nv <= 1) MOE_CBT(1);
  else if (nv <= 2) MOE_CBT(2);
  else if (nv <= 4) MOE_CBT(4);
  else return MOE_ERR_LIMIT;
#undef MOE_CBT
  return moe_launch_status();
}

extern "C" int moe_combine_bwd_by_token(const void* dy, int dy_dtype, const uint16_t* y,
                                        const float* gates, const int32_t* row_to_pos, int64_t T,
                                        int64_t H, int64_t k, uint16_t* dyp, float* dgates,
                                        void* stream) {
  if (T == 0) return 0;
  MOE_CHECK_PTR(dy);
  MOE_CHECK_PTR(dyp);
  if (y && !aligned16(y)) return MOE_ERR_ALIGN;
  if (!row_to_pos) return MOE_ERR_NULL;
  if ((dgates != nullptr) != (y != nullptr)) return MOE_ERR_NULL;
  if (T < 0 || H <= 0 || k <= 0 || (H % 8) != 0) return MOE_ERR_SHAPE;
  if (T * k > (int64_t)1 << 30 || H > 2048 || k > MOE_MAX_TOPK) return MOE_ERR_LIMIT;
  hipStream_t s = (hipStream_t)stream;
  if (dy_dtype == MOE_DT_BF16)
    return launch_combine_bwd_token<uint16_t>(dy, y, gates, row_to_pos, T, H, k, dyp, dgates, s);
  if (dy_dtype == MOE_DT_F32)
    return launch_combine_bwd_token<float>(dy, y, gates, row_to_pos, T, H, k, dyp, dgates, s);
  return MOE_ERR_DTYPE;
}

// dgates[r] = (sum_b part[b][row_to_pos[r]]) / gates[r]: the blocks hold gate * <dy, y> split
// over 64-column blocks of the intermediate width; a gate that underflowed to zero gets a zero
// gradient (the softmax Jacobian multiplies it by that gate again).
__global__ void dgates_from_blocks_kernel(const float* __restrict__ part, int P,
                                          const float* __restrict__ gates,
                                          const int32_t* __restrict__ row_to_pos, int R,
                                          float* __restrict__ dgates) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= R) return;
  const float* src = part + row_to_pos[r];
  float s = 0.f;
  for (int b = 0; b < P; ++b) s += src[(size_t)b * R];
  const float gt = gates[r];
  dgates[r] = gt != 0.f ? s / gt : 0.f;
}

// The same walk by position: the blocks of a position are read side by side with its neighbours'
// (coalesced), and only the result is scattered to the routed row (one 4-byte store and one
// 4-byte gate read per row instead of one scattered read per block and row).
__global__ void dgates_from_blocks_by_pos_kernel(const float* __restrict__ part, int P,
                                                 const float* __restrict__ gates,
                                                 const int32_t* __restrict__ pos_to_row, int R,
                                                 float* __restrict__ dgates) {
  const int pos = blockIdx.x * blockDim.x + threadIdx.x;
  if (pos >= R) return;
  float s = 0.f;
  for (int b = 0; b < P; ++b) s += part[(size_t)b * R + pos];
  const int r = pos_to_row[pos];
  const float gt = gates[r];
  dgates[r] = gt != 0.f ? s / gt : 0.f;
}

extern "C" int moe_dgates_from_blocks_by_pos(const float* part, int64_t P, const float* gates,
                                             const int32_t* pos_to_row, int64_t R, float* dgates,
                                             void* stream) {
  if (R == 0) return 0;
  if (!part || !gates || !pos_to_row || !dgates) return MOE_ERR_NULL;
  if (R < 0 || P <= 0) return MOE_ERR_SHAPE;
  if (R > (int64_t)1 << 30 || P > MAX_ROW_ELEMS) return MOE_ERR_LIMIT;
  hipLaunchKernelGGL(dgates_from_blocks_by_pos_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, part, (int)P, gates, pos_to_row, (int)R, dgates);
  return moe_launch_status();
}

extern "C" int moe_dgates_from_blocks(const float* part, int64_t P, const float* gates,
                                      const int32_t* row_to_pos, int64_t R, float* dgates,
                                      void* stream) {
  if (R == 0) return 0;
  if (!part || !gates || !row_to_pos || !dgates) return MOE_ERR_NULL;
  if (R < 0 || P <= 0) return MOE_ERR_SHAPE;
  if (R > (int64_t)1 << 30 || P > MAX_ROW_ELEMS) return MOE_ERR_LIMIT;
  hipLaunchKernelGGL(dgates_from_blocks_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, part, (int)P, gates, row_to_pos, (int)R, dgates);
  return moe_launch_status();
}

// seg[e*S + s] = offs[e] + (offs[e+1] - offs[e]) * s / S;  seg[E*S] = offs[E]
__global__ void segment_offsets_kernel(const int32_t* __restrict__ offs, int E, int S,
                                       int32_t* __restrict__ seg) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < E * S) {
    const int e = i / S, sidx = i % S;
    const long long lo = offs[e], len = offs[e + 1] - lo;
    seg[i] = (int32_t)(lo + len * sidx / S);
  } else if (i == E * S) {
    seg[i] = offs[E];
  }
}

extern "C" int moe_segment_offsets(const int32_t* offs, int64_t E, int64_t S, int32_t* seg,
                                   void* stream) {
  if (!offs || !seg) return MOE_ERR_NULL;
  if (E <= 0 || S <= 0) return MOE_ERR_SHAPE;
  if (E * S > 1024) return MOE_ERR_LIMIT;
  const int n = (int)(E * S + 1);
  hipLaunchKernelGGL(segment_offsets_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                     offs, (int)E, (int)S, seg);
  return moe_launch_status();
}

// Row segments of at most L rows each: expert e is cut into ceil(n_e / L) equal parts, numbered
// expert by expert.  seg_start[e] = index of e's first segment (seg_start[E] = their number);
// seg[s] = first row of segment s; the slots past the last used one, up to S_max, are empty
// segments at the end of the rows.  One wave: a scan over the experts' segment counts.
__global__ void segments_by_length_kernel(const int32_t* __restrict__ offs, int E, int L, int S_max,
                                          int32_t* __restrict__ seg, int32_t* __restrict__ seg_start) {
  const int lane = threadIdx.x;
  int carry = 0;
  for (int b = 0; b < E; b += MOE_WAVE) {
    const int e = b + lane;
    const int lo = e < E ? offs[e] : 0;
    const int n = e < E ? offs[e + 1] - lo : 0;
    const int ns = (n + L - 1) / L;
    int incl = ns;
#pragma unroll
    for (int off = 1; off < MOE_WAVE; off <<= 1) {
      const int o = __shfl_up(incl, off, MOE_WAVE);
      if (lane >= off) incl += o;
    }
    const int start = carry + incl - ns;
    if (e < E) {
      seg_start[e] = start;
      for (int j = 0; j < ns; ++j) seg[start + j] = lo + (int32_t)((long long)n * j / ns);
    }
    carry += __shfl(incl, MOE_WAVE - 1, MOE_WAVE);
  }
  if (lane == 0) seg_start[E] = carry;
  const int R = offs[E];
  for (int s2 = carry + lane; s2 <= S_max; s2 += MOE_WAVE) seg[s2] = R;
}

extern "C" int64_t moe_segments_by_length_max(int64_t R, int64_t E, int64_t L) {
  if (R < 0 || E <= 0 || L <= 0) return 0;
  return (R + L - 1) / L + E;
}

extern "C" int moe_segment_offsets_by_length(const int32_t* offs, int64_t E, int64_t L, int64_t S_max,
                                             int32_t* seg, int32_t* seg_start, void* stream) {
  if (!offs || !seg || !seg_start) return MOE_ERR_NULL;
  if (E <= 0 || L <= 0 || S_max < E) return MOE_ERR_SHAPE;
  if (E > 1024 || S_max > 1024 || L > (int64_t)1 << 30) return MOE_ERR_LIMIT;
  hipLaunchKernelGGL(segments_by_length_kernel, dim3(1), dim3(MOE_WAVE), 0, (hipStream_t)stream, offs,
                     (int)E, (int)L, (int)S_max, seg, seg_start);
  return moe_launch_status();
}

// dw[e] (+)= sum of part[s] over e's segments in ascending order; 8 elements per thread.
template <typename OutT>
__global__ void reduce_segments_kernel(const float* __restrict__ part, const int32_t* __restrict__ seg_start,
                                       int E, long long mn8, OutT* __restrict__ dw, int accumulate) {
  const long long total = (long long)E * mn8;
  for (long long idx = blockIdx.x * (long long)blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const int e = (int)(idx / mn8);
    const long long i = idx - (long long)e * mn8;
    const int s0 = seg_start[e], s1 = seg_start[e + 1];
    Row8 acc;
#pragma unroll
    for (int v = 0; v < 8; ++v) acc.v[v] = 0.f;
    for (int sg = s0; sg < s1; ++sg) {
      const Row8 r = load8(part + ((long long)sg * mn8 + i) * 8);
#pragma unroll
      for (int v = 0; v < 8; ++v) acc.v[v] += r.v[v];
    }
    OutT* dst = dw + idx * 8;
    if (accumulate) {
      const Row8 old = load8(dst);
#pragma unroll
      for (int v = 0; v < 8; ++v) acc.v[v] += old.v[v];
    }
    store8(dst, acc);
  }
}

extern "C" int moe_wgrad_reduce_segments(const float* part, const int32_t* seg_start, int64_t E, int64_t M,
                                         int64_t N, void* dw, int dw_dtype, int accumulate, void* stream) {
  if (!seg_start) return MOE_ERR_NULL;
  if (E <= 0 || M <= 0 || N <= 0 || (M % 8) || (N % 8)) return MOE_ERR_SHAPE;
  if (E > 1024 || M > (1 << 16) || N > (1 << 16)) return MOE_ERR_LIMIT;
  MOE_CHECK_PTR(part);
  MOE_CHECK_PTR(dw);
  const long long mn8 = M * N / 8;
  long long blocks = (E * mn8 + 255) / 256;
  if (blocks > 256 * 8) blocks = 256 * 8;
  hipStream_t st = (hipStream_t)stream;
  if (dw_dtype == MOE_DT_F32)
    hipLaunchKernelGGL(reduce_segments_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st, part, seg_start,
                       (int)E, mn8, (float*)dw, accumulate);
  else if (dw_dtype == MOE_DT_BF16)
    hipLaunchKernelGGL(reduce_segments_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, st, part, seg_start,
                       (int)E, mn8, (uint16_t*)dw, accumulate);
  else
    return MOE_ERR_DTYPE;
  return moe_launch_status();
}

extern "C" int moe_cast_f32_bf16(const float* src, uint16_t* dst, int64_t n, void* stream) {
  if (n == 0) return 0;
  MOE_CHECK_PTR(src);
  MOE_CHECK_PTR(dst);
  if (n < 0) return MOE_ERR_SHAPE;
  const long long n8 = n / 8;
  long long blocks = (n8 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(cast_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, src,
                     dst, n8, (long long)n);
  return moe_launch_status();
}
