// Grouped (per-expert, ragged) bf16 GEMMs on the gfx950 matrix cores.
//
// One kernel template covers the five products of the expert FFN and its backward.  All of
// them are   C[rows, cols] = sum_k A[rows, k] * B[cols, k]   computed per expert with
// v_mfma_f32_32x32x16_bf16 (fp32 accumulation); they differ in which dimension is ragged,
// in how the operands lie in memory, and in the epilogue:
//
//   GATEUP        rows = expert's tokens, k = H.  A = xp [R,H]; B = W1 and W3 [E,I,H] (two
//                 accumulator sets share every A fragment); epilogue act = silu(g)*u.
//   DOWN          rows = tokens, k = I.  A = act [R,I]; B = W2 [E,H,I].
//   DGRAD_DOWN    rows = tokens, k = H.  A = dy [R,H]; B = W2 [E,H,I] read as [k][col];
//                 epilogue dg = dact*u*silu'(g), du = dact*silu(g).
//   DGRAD_GATEUP  rows = tokens, k runs over two segments of I.  A = dg | du [R,I];
//                 B = W1 | W3 [E,I,H] read as [k][col].
//   WGRAD         k = expert's tokens (ragged).  A = a [R,M] and B = b [R,N], both read as
//                 [k][row]; C = dw[e] [M,N].
//
// Memory plan.  A workgroup owns one BM x BN output tile.  A and B tiles of depth BK travel
// HBM -> registers (buffer loads whose hardware bounds check returns zero past the end of
// the expert's rows, so ragged tails cost no instructions) -> LDS (two stages) -> MFMA
// operand fragments.  The loop is software-pipelined: while the MFMAs of k-step s run, the
// fragments of step s+1 are read from LDS, the tile for iteration t+1 is written to the
// other LDS stage and the tile for iteration t+2 is requested from HBM.  There is one
// workgroup barrier per iteration, placed before the last k-step so that the first
// fragment reads of the next stage hide behind that step's MFMAs.
// Operands that are k-contiguous in memory are kept k-contiguous in LDS (16-byte fragment
// reads, rows padded by 16 bytes against bank conflicts); operands that are not are kept
// as they lie in memory and read through the transposing LDS read of gfx950.
// Workgroups are numbered so that each XCD (own L2) works on a contiguous range of tiles,
// i.e. on its own experts' weights.
#include "common.h"

namespace {

enum Mode { GATEUP = 0, DOWN = 1, DGRAD_DOWN = 2, DGRAD_GATEUP = 3, WGRAD = 4 };

struct GemmArgs {
  const uint16_t* A0;
  const uint16_t* A1;
  const uint16_t* B0;
  const uint16_t* B1;
  void* C0;
  void* C1;
  void* C2;
  const uint16_t* X0;
  const uint16_t* X1;
  const int32_t* offs;
  int E;        // experts
  int R;        // total rows of the row-ragged operand(s)
  int M;        // WGRAD only: rows of dw[e]
  int N;        // output columns
  int K;        // contraction length per segment (not used by WGRAD)
  int n_tiles;  // tiles along N
  int m_slots;  // row-tile slots (ragged modes) or tiles along M (WGRAD)
  int accumulate;
  int ld_a;     // row stride of A0/A1 in elements when it is not the contraction length (0: K)
  int ld_c;     // row stride of the outputs C0/C1 in elements when it is not N (0: N)
  int m_split;  // WGRAD: rows m >= m_split of an expert's result go to C1 (as its rows m - m_split); 0: all to C0
};

template <int BM_, int BN_, int BK_, int WM_, int WN_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_;
  static constexpr int NT = WM * WN * MOE_WAVE;
  static constexpr int WTM = BM / WM, WTN = BN / WN;
  static constexpr int FM = WTM / 32, FN = WTN / 32;
  static constexpr int KS = BK / 16;
  // workgroups meant to share a CU (their LDS footprints must fit together in 160 KB)
  static constexpr int WGS_PER_CU = (NT >= 512) ? 1 : 2;
  static constexpr int WAVES_PER_SIMD = NT / 256 * WGS_PER_CU;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 32 == 0, "tile shape");
};

// sigmoid from the two hardware transcendentals (v_exp_f32, v_rcp_f32; about 1 ulp each):
// the epilogues are VALU-bound, and an IEEE division would triple their cost.
__device__ __forceinline__ float sigmoidf_(float x) {
  return __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

// A window of global memory read through a buffer resource: reads at or past `bytes`
// return zero.  Only the per-lane offset takes part in the hardware bounds check (a scalar
// offset does not), so a window is advanced along k by moving its base and shrinking its
// size, both scalar operations.
struct View {
  const uint16_t* base;
  long long bytes;
};
__device__ __forceinline__ View make_view(const uint16_t* base, long long valid_elems) {
  return View{base, valid_elems > 0 ? valid_elems * 2 : 0};
}
__device__ __forceinline__ __amdgpu_buffer_rsrc_t view_rsrc(const View& w, long long byte_off) {
  long long left = w.bytes - byte_off;
  if (left < 0) left = 0;
  if (left > 0xffffffffll) left = 0xffffffffll;
  return __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)w.base + byte_off), 0,
                                           (int)(unsigned)left, 0x00020000);
}

// ---- operand staging ----------------------------------------------------------------------
// Two LDS layouts, one per memory order of the operand, each with the fragment read that
// hands an MFMA lane its 8 consecutive k values for row (lane % 32):
//
// OpInner  source is k-contiguous: element (r, kk) at view[r * ld + k0 + kk].
//          LDS holds [ROWS][BK + 8] (16 bytes of padding per row); a fragment is one
//          16-byte LDS read.
// OpOuter  source is row-contiguous: element (r, kk) at view[(k0 + kk) * ld + r].
//          LDS holds the tile as it lies in memory, [BK][ROWS + 32] (64 bytes of padding
//          per k line); a fragment is two ds_read_b64_tr_b16, the gfx950 transposing LDS
//          read: a group of 16 lanes addresses a block of 4 k lines x 16 columns (lane i
//          points at line i/4, columns 4*(i%4)..+3) and lane i gets back column i of that
//          block, i.e. 4 consecutive k of its own row.
template <int ROWS_, int BK, int NT>
struct OpInner {
  static constexpr int ROWS = ROWS_;
  static constexpr int LDK = BK + 8;
  static constexpr int LDS_ELEMS = ROWS * LDK;
  static constexpr int CPR = BK / 8;          // 16-byte chunks per row
  static constexpr int CH = ROWS * CPR / NT;  // chunks per thread
  static constexpr int RSTEP = NT / CPR;      // rows between a thread's consecutive chunks
  static_assert((ROWS * CPR) % NT == 0 && NT % CPR == 0, "loader shape");
  int voff[CH];  // byte offsets of this thread's chunks inside the view at k0 = 0
  int lds_w;     // element offset of its first chunk in the LDS tile
  int kc;        // first k of its chunks inside the tile
  __device__ __forceinline__ void init(int ld) {
    const int r = threadIdx.x / CPR;
    kc = (threadIdx.x % CPR) * 8;
#pragma unroll
    for (int i = 0; i < CH; ++i) voff[i] = ((r + i * RSTEP) * ld + kc) * 2;
    lds_w = r * LDK + kc;
  }
  static __device__ __forceinline__ long long k_bytes(int k0, int /*ld*/) { return (long long)k0 * 2; }
  __device__ __forceinline__ u32x4 load_one(int i, __amdgpu_buffer_rsrc_t rs) const {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, voff[i], 0, 0);
  }
  // k beyond the end of the contraction lies in the next row of a k-contiguous source, so
  // the hardware bound cannot catch it: such chunks are cleared by hand (k_left = valid k)
  __device__ __forceinline__ bool past_k(int k_left) const { return kc >= k_left; }
  __device__ __forceinline__ void store_one(int i, uint16_t* lds, u32x4 v) const {
    *reinterpret_cast<u32x4*>(lds + lds_w + i * RSTEP * LDK) = v;
  }
  static __device__ __forceinline__ int lane_off(int lane) { return (lane & 31) * LDK + (lane >> 5) * 8; }
  static __device__ __forceinline__ bf16x8 frag(const uint16_t* lds, int lane_offset, int row_base, int ks) {
    return *reinterpret_cast<const bf16x8*>(lds + lane_offset + row_base * LDK + ks * 16);
  }
};

template <int ROWS_, int BK, int NT>
struct OpOuter {
  static constexpr int ROWS = ROWS_;
  static constexpr int LDN = ROWS + 32;
  static constexpr int LDS_ELEMS = BK * LDN;
  static constexpr int CPK = ROWS / 8;        // 16-byte chunks per k line
  static constexpr int CH = BK * CPK / NT;
  static constexpr int KSTEP = NT / CPK;      // k lines between a thread's consecutive chunks
  static_assert((BK * CPK) % NT == 0 && NT % CPK == 0, "loader shape");
  int voff[CH];
  int lds_w;
  __device__ __forceinline__ void init(int ld) {
    const int kk = threadIdx.x / CPK, rc = (threadIdx.x % CPK) * 8;
#pragma unroll
    for (int i = 0; i < CH; ++i) voff[i] = ((kk + i * KSTEP) * ld + rc) * 2;
    lds_w = kk * LDN + rc;
  }
  static __device__ __forceinline__ long long k_bytes(int k0, int ld) { return (long long)k0 * ld * 2; }
  __device__ __forceinline__ u32x4 load_one(int i, __amdgpu_buffer_rsrc_t rs) const {
    return __builtin_amdgcn_raw_buffer_load_b128(rs, voff[i], 0, 0);
  }
  // the k bound of this layout is the end of the view: the hardware zero-fills
  __device__ __forceinline__ bool past_k(int) const { return false; }
  __device__ __forceinline__ void store_one(int i, uint16_t* lds, u32x4 v) const {
    *reinterpret_cast<u32x4*>(lds + lds_w + i * KSTEP * LDN) = v;
  }
  // lane l = 16*b + i: k line (b/2)*8 + i/4, columns 16*(b%2) + 4*(i%4) .. +3
  static __device__ __forceinline__ int lane_off(int lane) {
    const int i = lane & 15, b = lane >> 4;
    return ((b >> 1) * 8 + (i >> 2)) * LDN + (b & 1) * 16 + (i & 3) * 4;
  }
  static __device__ __forceinline__ bf16x8 frag(const uint16_t* lds, int lane_offset, int row_base, int ks) {
    const uint16_t* p = lds + lane_offset + ks * 16 * LDN + row_base;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p + 4 * LDN));
    typedef __attribute__((ext_vector_type(8))) short s16x8;
    const s16x8 r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, r);
  }
};

// Wait for this wave's LDS traffic, then meet the other waves.  Global loads stay in flight.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int MODE, typename Cfg>
constexpr int lds_bytes() {
  constexpr bool a_outer = (MODE == WGRAD);
  constexpr bool b_outer = (MODE == DGRAD_DOWN || MODE == DGRAD_GATEUP || MODE == WGRAD);
  constexpr int a = a_outer ? OpOuter<Cfg::BM, Cfg::BK, Cfg::NT>::LDS_ELEMS : OpInner<Cfg::BM, Cfg::BK, Cfg::NT>::LDS_ELEMS;
  constexpr int b = b_outer ? OpOuter<Cfg::BN, Cfg::BK, Cfg::NT>::LDS_ELEMS : OpInner<Cfg::BN, Cfg::BK, Cfg::NT>::LDS_ELEMS;
  return 2 * (a + b) * 2;
}

constexpr int GEMM_MAX_E = 1024;  // per-expert tile prefix lives in LDS

// BLK (GATEUP and DGRAD_DOWN only): g and u, which nothing but the SwiGLU backward reads, are kept
// in a layout private to the library instead of as [R, I] rows: one 4 KB record per 32 x 32 block
// of a row tile, holding the block exactly as the matrix cores leave it in a wave's accumulators
// (see gu_block below).  The forward kernel then stores them straight from its registers and the
// backward kernel loads them straight into the layout it computes in: neither passes them
// through LDS.
template <int MODE, typename Cfg, typename OutT, bool BLK = false>
__global__ __launch_bounds__(Cfg::NT, Cfg::WAVES_PER_SIMD) void grouped_gemm_kernel(const GemmArgs p) {
  static_assert(!BLK || MODE == GATEUP || MODE == DGRAD_DOWN, "only g and u have the blocked layout");
  constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, NT = Cfg::NT, KS = Cfg::KS;
  constexpr int FM = Cfg::FM, FN = Cfg::FN, WTM = Cfg::WTM, WTN = Cfg::WTN;
  constexpr bool DUAL = (MODE == GATEUP);
  constexpr int BNC = DUAL ? BN / 2 : BN;  // output columns covered by the tile
  constexpr bool A_OUTER = (MODE == WGRAD);
  constexpr bool B_OUTER = (MODE == DGRAD_DOWN || MODE == DGRAD_GATEUP || MODE == WGRAD);
  constexpr int NSEG = (MODE == DGRAD_GATEUP) ? 2 : 1;
  static_assert(!DUAL || (FN % 2 == 0), "dual mode needs an even number of column fragments");
  static_assert(KS % 2 == 0, "fragment double buffering assumes an even number of k-steps");

  using StA = typename std::conditional<A_OUTER, OpOuter<BM, BK, NT>, OpInner<BM, BK, NT>>::type;
  using StB = typename std::conditional<B_OUTER, OpOuter<BN, BK, NT>, OpInner<BN, BK, NT>>::type;
  using StBh = OpInner<BN / 2, BK, NT>;  // dual mode: the W1 half and the W3 half of the B tile
  static_assert(!DUAL || !B_OUTER, "dual mode stages k-contiguous weights");

  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  __shared__ int tile_start[(MODE == WGRAD) ? 1 : GEMM_MAX_E + 1];
  uint16_t* sA = smem;                       // [2][StA::LDS_ELEMS]
  uint16_t* sB = smem + 2 * StA::LDS_ELEMS;  // [2][StB::LDS_ELEMS]

  // (the wave's index is the same in all of its lanes: read it once so that everything derived
  // from it lives in scalar registers)
  const int lane = threadIdx.x & 63, wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wm = wv / Cfg::WN, wn = wv % Cfg::WN;

  // ---- which tiles this workgroup computes
  // The kernel is persistent: the grid has one workgroup per compute unit and each walks a
  // list of tiles.  Hardware hands workgroup b to XCD b % 8 (each XCD has its own L2), so
  // XCD x takes the x-th contiguous eighth of the tile list and its workgroups sweep that
  // range side by side: at any time they share a few experts' weights and row blocks in L2.
  if constexpr (MODE != WGRAD) {
    // tile_start[e] = number of row tiles of the experts before e (wave 0 scans)
    if (threadIdx.x < MOE_WAVE) {
      int carry = 0;
      for (int b = 0; b < p.E; b += MOE_WAVE) {
        const int e = b + lane;
        const int nt = e < p.E ? (p.offs[e + 1] - p.offs[e] + BM - 1) / BM : 0;
        int incl = nt;
#pragma unroll
        for (int off = 1; off < MOE_WAVE; off <<= 1) {
          const int o = __shfl_up(incl, off, MOE_WAVE);
          if (lane >= off) incl += o;
        }
        if (e < p.E) tile_start[e] = carry + incl - nt;
        carry += __shfl(incl, MOE_WAVE - 1, MOE_WAVE);
      }
      if (lane == 0) tile_start[p.E] = carry;
    }
    __syncthreads();
  }
  // The XCDs that have workgroups (all 8 unless the grid is tiny) share out the tile list.
  // Row-ragged modes: every tile costs about the same; XCD x takes the x-th contiguous eighth of
  // the list (equal counts of real tiles) and its workgroups sweep it side by side.
  // WGRAD with more tiles than workgroups: a tile of expert e contracts over that expert's rows,
  // so under skewed routing tiles differ in cost by orders of magnitude and a contiguous range is
  // all heavy or all light.  The (expert-major) list is dealt in groups of as many consecutive
  // tiles as an XCD has workgroups, group g to XCD g % 8, one tile to each of its workgroups: the
  // workgroups of an XCD stay on one expert (or two) and walk its rows together, and every XCD
  // sees every part of the list.  With at most 64 experts, whole groups per expert and skewed
  // routing (the largest expert above 1.25 times the mean) the groups are not dealt round-robin
  // but longest first: experts in descending order of their rows, each group to the XCD with the
  // least work so far; every workgroup works that out for itself from the offsets, the same way,
  // and keeps its own tiles' numbers in LDS.  (A generated power-law skew over 16 experts: 10-12 %
  // faster dealt in groups than with contiguous ranges of equal work, another 9-10 % longest
  // first; near-uniform routing: the same in all three.)
  constexpr int MAX_GROUPS = 512;
  __shared__ int glist[(MODE == WGRAD) ? MAX_GROUPS : 1];
  __shared__ int gcount;
  int t_next, t_hi, t_step;  // (t_step == 0: positions in glist, else tile numbers)
  {
    const int nb = gridDim.x, x = blockIdx.x & 7, j = blockIdx.x >> 3;
    const int nx = nb < 8 ? nb : 8;
    t_step = (nb >> 3) + (x < (nb & 7) ? 1 : 0);
    int lo;
    if (MODE == WGRAD && p.E * p.m_slots * p.n_tiles > nb && (nb & 7) == 0) {
      const int wgs = nb >> 3, TP = p.m_slots * p.n_tiles;
      lo = x * wgs;
      t_hi = p.E * TP;
      t_step = nb;
      if (p.E <= MOE_WAVE && TP % wgs == 0 && p.E * (TP / wgs) <= MAX_GROUPS) {
        if (threadIdx.x < MOE_WAVE) {
          const int gpe = TP / wgs;  // groups per expert
          constexpr long long FIXED = 4 * BK;  // fill, tile switch and epilogue, in rows' worth
          int rows = 0;
          if (lane < p.E) {
            rows = p.offs[lane + 1] - p.offs[lane];
            rows = rows < 0 ? 0 : rows;
          }
          const long long cost = rows + FIXED;
          // (only worth it when the routing is skewed: with near-equal experts the plain dealing is
          // as balanced and keeps neighbouring experts on neighbouring XCDs)
          int mx = rows, sum = rows;
#pragma unroll
          for (int off = MOE_WAVE / 2; off > 0; off >>= 1) {
            const int om = __shfl_xor(mx, off, MOE_WAVE);
            mx = om > mx ? om : mx;
            sum += __shfl_xor(sum, off, MOE_WAVE);
          }
          const bool skewed = 4ll * mx * p.E > 5ll * sum;
          int rank = 0;  // position of expert `lane` in descending order of cost (ties: lower index first)
          for (int o = 0; o < p.E; ++o) {
            const long long co = __shfl(cost, o, MOE_WAVE);
            rank += (co > cost || (co == cost && o < lane)) ? 1 : 0;
          }
          if (lane >= p.E) rank = -1;
          // lanes 0..7 carry the XCDs' loads, packed with the XCD index for the arg-min
          long long load = 0;
          int cnt = 0;
          for (int s_ = 0; skewed && s_ < p.E; ++s_) {
            const int e = __builtin_ctzll(__ballot(rank == s_));
            const long long ce = __shfl(cost, e, MOE_WAVE);
            for (int gi = 0; gi < gpe; ++gi) {
              long long key = lane < 8 ? ((load << 3) | lane) : 0x7fffffffffffffffll;
#pragma unroll
              for (int off = 1; off < 8; off <<= 1) {
                const long long other = __shfl_xor(key, off, MOE_WAVE);
                key = other < key ? other : key;
              }
              const int xmin = (int)(__shfl(key, 0, MOE_WAVE) & 7);
              if (lane == xmin) load += ce;
              if (xmin == x) {
                if (lane == 0) glist[cnt] = (e * gpe + gi) * wgs + j;
                ++cnt;
              }
            }
          }
          if (lane == 0) gcount = skewed ? cnt : -1;
        }
        __syncthreads();
        const int cnt = gcount;
        if (cnt >= 0) {
          t_hi = cnt;  // (positions in the list)
          lo = -j;
          t_step = 0;
        }
      }
    } else {
      int total;  // real tiles
      if constexpr (MODE == WGRAD) total = p.E * p.m_slots * p.n_tiles;
      else total = tile_start[p.E] * p.n_tiles;
      const int q = total / nx, r = total % nx;
      lo = x * q + (x < r ? x : r);
      t_hi = lo + q + (x < r ? 1 : 0);
    }
    t_next = lo + j;
  }
  // the tile behind position `pos` of this workgroup's walk
  auto tile_at = [&](int pos) { return t_step == 0 ? __builtin_amdgcn_readfirstlane(glist[pos]) : pos; };

  struct Tile {
    int e, row0, row_end, n0, m0, slot;
    int Kseg, kt_per_seg, nkt;
    bool need_mask;
    View vA0, vA1, vB0, vB1;
  };
  int lda, ldb;
  if constexpr (MODE == GATEUP || MODE == DOWN) lda = ldb = p.K;
  else if constexpr (MODE == WGRAD) { lda = p.M; ldb = p.N; }
  else { lda = p.ld_a ? p.ld_a : p.K; ldb = p.N; }

  // Fills `t` for tile slot `logical`; false when the slot lies past the last real tile.
  // Every lane computes the same thing from the same LDS words / scalar loads.
  auto locate = [&](int logical, Tile& t) -> bool {
    const int n_tile = logical % p.n_tiles;
    const int slot = logical / p.n_tiles;
    t.m0 = 0;
    t.slot = slot;
    if constexpr (MODE == WGRAD) {
      t.e = slot / p.m_slots;
      t.m0 = (slot % p.m_slots) * BM;
      t.row0 = p.offs[t.e];
      t.row_end = p.offs[t.e + 1];
    } else {
      if (slot >= tile_start[p.E]) return false;
      int lo = 0, hi = p.E;  // largest e with tile_start[e] <= slot (skips empty experts)
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (tile_start[mid] <= slot) lo = mid;
        else hi = mid;
      }
      t.e = __builtin_amdgcn_readfirstlane(lo);
      t.row0 = p.offs[t.e] + (slot - __builtin_amdgcn_readfirstlane(tile_start[lo])) * BM;
      t.row_end = p.offs[t.e + 1];
    }
    t.n0 = n_tile * BNC;
    t.Kseg = (MODE == WGRAD) ? (t.row_end - t.row0) : p.K;
    t.kt_per_seg = (t.Kseg + BK - 1) / BK;
    t.nkt = t.kt_per_seg * NSEG;
    // k-contiguous operands whose contraction length is not a multiple of BK need their
    // last k-tile cleared by hand; that path gives up the static schedule (never taken
    // when H and I are multiples of BK)
    t.need_mask = ((t.Kseg % BK) != 0) && (!A_OUTER || !B_OUTER);
    const long long rows = t.row_end - t.row0;
    if constexpr (MODE == GATEUP) {
      t.vA0 = make_view(p.A0 + (long long)t.row0 * lda, rows * lda);
      const long long wofs = ((long long)t.e * p.N + t.n0) * p.K;
      const long long wvalid = (long long)(p.N - t.n0) * p.K;
      t.vB0 = make_view(p.B0 + wofs, wvalid);
      t.vB1 = make_view(p.B1 + wofs, wvalid);
    } else if constexpr (MODE == DOWN) {
      t.vA0 = make_view(p.A0 + (long long)t.row0 * lda, rows * lda);
      t.vB0 = make_view(p.B0 + ((long long)t.e * p.N + t.n0) * p.K, (long long)(p.N - t.n0) * p.K);
    } else if constexpr (MODE == DGRAD_DOWN || MODE == DGRAD_GATEUP) {
      // A = dy [R,K] (or dg|du [R,K]); B = W[e] as [K][N]
      t.vA0 = make_view(p.A0 + (long long)t.row0 * lda, rows * lda);
      t.vB0 = make_view(p.B0 + (long long)t.e * p.K * p.N + t.n0, (long long)p.K * p.N - t.n0);
      if constexpr (MODE == DGRAD_GATEUP) {
        t.vA1 = make_view(p.A1 + (long long)t.row0 * lda, rows * lda);
        t.vB1 = make_view(p.B1 + (long long)t.e * p.K * p.N + t.n0, (long long)p.K * p.N - t.n0);
      }
    } else {  // WGRAD: A = a [R,M] as [k][m]; B = b [R,N] as [k][n]; k = rows of expert e
      t.vA0 = make_view(p.A0 + (long long)t.row0 * lda + t.m0, rows * lda - t.m0);
      t.vB0 = make_view(p.B0 + (long long)t.row0 * ldb + t.n0, rows * ldb - t.n0);
    }
    return true;
  };

  // ---- loader addressing (the same for every tile) and staging registers
  StA opA;
  StB opB;
  StBh opB0, opB1;
  opA.init(lda);
  if constexpr (DUAL) {
    opB0.init(ldb);
    opB1.init(ldb);
  } else {
    opB.init(ldb);
  }
  // One set of registers carries a k-tile from HBM to LDS: it is requested one iteration
  // before it is written to LDS, which is what hides the latency of a load that misses L2.
  constexpr int CHA = StA::CH, CHB = DUAL ? StBh::CH : StB::CH;
  constexpr int NCH = CHA + (DUAL ? 2 : 1) * CHB;  // 16-byte chunks per thread per k-tile
  struct Stage {
    u32x4 v[NCH];
  };
  Stage stg;
  struct TileSrc {
    __amdgpu_buffer_rsrc_t a, b0, b1;
    int k_left;
  };
  auto tile_src = [&](const Tile& t, int kt) {
    const int seg = (NSEG == 2) ? kt / t.kt_per_seg : 0;
    const int k0 = (kt - seg * t.kt_per_seg) * BK;
    TileSrc ts;
    ts.a = view_rsrc((NSEG == 2 && seg) ? t.vA1 : t.vA0, StA::k_bytes(k0, lda));
    if constexpr (DUAL) {
      ts.b0 = view_rsrc(t.vB0, StBh::k_bytes(k0, ldb));
      ts.b1 = view_rsrc(t.vB1, StBh::k_bytes(k0, ldb));
    } else {
      ts.b0 = view_rsrc((NSEG == 2 && seg) ? t.vB1 : t.vB0, StB::k_bytes(k0, ldb));
      ts.b1 = ts.b0;
    }
    ts.k_left = t.Kseg - k0;
    return ts;
  };
  auto load_chunk = [&](int c, Stage& st, const TileSrc& ts) {
    if (c < CHA) st.v[c] = opA.load_one(c, ts.a);
    else if constexpr (DUAL) {
      if (c < CHA + CHB) st.v[c] = opB0.load_one(c - CHA, ts.b0);
      else st.v[c] = opB1.load_one(c - CHA - CHB, ts.b1);
    } else {
      st.v[c] = opB.load_one(c - CHA, ts.b0);
    }
  };
  auto clear_past_k = [&](int c, Stage& st, int k_left) {
    bool past;
    if (c < CHA) past = opA.past_k(k_left);
    else if constexpr (DUAL) past = opB0.past_k(k_left);
    else past = opB.past_k(k_left);
    if (past) st.v[c] = u32x4{0, 0, 0, 0};
  };
  auto store_chunk = [&](int c, const Stage& st, int buf) {
    if (c < CHA) opA.store_one(c, sA + buf * StA::LDS_ELEMS, st.v[c]);
    else if constexpr (DUAL) {
      if (c < CHA + CHB) opB0.store_one(c - CHA, sB + buf * StB::LDS_ELEMS, st.v[c]);
      else opB1.store_one(c - CHA - CHB, sB + buf * StB::LDS_ELEMS + StBh::LDS_ELEMS, st.v[c]);
    } else {
      opB.store_one(c - CHA, sB + buf * StB::LDS_ELEMS, st.v[c]);
    }
  };
  auto load_tile = [&](const Tile& t, int kt, Stage& st) {
    const TileSrc ts = tile_src(t, kt);
#pragma unroll
    for (int c = 0; c < NCH; ++c) load_chunk(c, st, ts);
    if (t.need_mask && ts.k_left < BK) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) clear_past_k(c, st, ts.k_left);
    }
  };
  auto store_tile = [&](const Stage& st, int buf) {
#pragma unroll
    for (int c = 0; c < NCH; ++c) store_chunk(c, st, buf);
  };
  using std::integral_constant;
  const int a_off = StA::lane_off(lane), b_off = StB::lane_off(lane);
  // LDS row of column-fragment jn for this wave
  auto bfrag_row = [&](int jn) {
    if constexpr (DUAL)
      return (jn < FN / 2) ? wn * (WTN / 2) + jn * 32 : BN / 2 + wn * (WTN / 2) + (jn - FN / 2) * 32;
    else
      return wn * WTN + jn * 32;
  };

  struct Frags {
    bf16x8 a[FM];
    bf16x8 b[FN];
  };
  f32x16 acc[FM][FN];
  Frags fr[2];
  constexpr int NMMA = FM * FN;  // MFMAs per k-step
  constexpr int NFR = FM + FN;   // fragment reads per k-step
  // u-th fragment read of a k-step: a0, b0 .. b(FN-1), a1 .. a(FM-1) -- the order in which
  // the MFMAs (row-major over the fragment grid) first need them
  auto f_read_one = [&](int u, int buf, int ks, Frags& f) {
    const uint16_t* a_lds = sA + buf * StA::LDS_ELEMS;
    const uint16_t* b_lds = sB + buf * StB::LDS_ELEMS;
    if (u == 0) f.a[0] = StA::frag(a_lds, a_off, wm * WTM, ks);
    else if (u <= FN) f.b[u - 1] = StB::frag(b_lds, b_off, bfrag_row(u - 1), ks);
    else f.a[u - FN] = StA::frag(a_lds, a_off, wm * WTM + (u - FN) * 32, ks);
  };
  auto mma_one = [&](int n, const Frags& f) {
    // boustrophedon over the fragment grid: consecutive MFMAs share one operand register (about
    // half a percent on every mode, measured); operands swapped: acc holds the transposed block
    const int i = n / FN, j = (i & 1) ? FN - 1 - n % FN : n % FN;
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.b[j], f.a[i], acc[i][j], 0, 0, 0);
  };
  auto f_read_all = [&](int buf, int ks, Frags& f) {
#pragma unroll
    for (int u = 0; u < NFR; ++u) f_read_one(u, buf, ks, f);
  };
  auto mma_all = [&](const Frags& f) {
#pragma unroll
    for (int n = 0; n < NMMA; ++n) mma_one(n, f);
  };

  // ---- one steady-state iteration, written out instruction by instruction: each MFMA is
  // followed by at most one chunk hand-over (registers -> LDS, then the same registers are
  // re-requested from HBM for the tile after next) and one fragment read, and a scheduling
  // fence after each slot keeps the compiler from clumping them, so a wave issues its
  // memory traffic in the shadow of its own MFMAs.
  //   phases 0..KS-2  MFMAs of k-step s | chunks of tile kt+1 -> other LDS stage, chunks of
  //                   tile kt+2 requested | fragments of step s+1 read
  //   last phase      barrier (stage kt fully read, stage kt+1 fully written) | MFMAs of the
  //                   last step | first fragment reads of stage kt+1 hide behind them
  auto body = [&](auto par_c, const Tile& t, int kt) {
    constexpr int buf = decltype(par_c)::value;  // LDS stage of k-tile kt == parity of kt
    Stage& st = stg;                             // holds k-tile kt+1, refilled with kt+2
    const TileSrc ts = tile_src(t, kt + 2);
    constexpr int NSLOT = (KS - 1) * NMMA;  // MFMA slots before the barrier
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
#pragma unroll
      for (int n = 0; n < NMMA; ++n) {
        mma_one(n, fr[ks & 1]);
        const int slot = ks * NMMA + n;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
          if (c * NSLOT / NCH == slot) {
            store_chunk(c, st, buf ^ 1);
            load_chunk(c, st, ts);
          }
        }
        if (n < NFR) f_read_one(n, buf, ks + 1, fr[(ks + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    lds_barrier();
#pragma unroll
    for (int n = 0; n < NMMA; ++n) {
      mma_one(n, fr[(KS - 1) & 1]);
      if (n < NFR) f_read_one(n, buf ^ 1, 0, fr[0]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- epilogue pieces.  The MFMAs were issued with the operands swapped (B fragment
  // first), so acc[i][j] holds the transposed 32x32 block: lane l owns output row (l % 32)
  // and, for q = 0..3, the four consecutive columns 8*q + 4*(l/32) .. +3 in
  // acc[i][j][4*q .. 4*q+3].  Results leave through LDS: each wave owns a strip of 32 rows
  // x its output columns, writes its accumulators there four columns at a time and reads
  // the strip back row-wise, so that global memory sees 16-byte stores that cover whole
  // 128-byte lines.  The strips live in the (then idle) operand stages, one region per
  // wave, so only wave-local ordering is needed between the two barriers that fence the
  // epilogue off from the main loops before and after it.
  constexpr int WTNC = DUAL ? WTN / 2 : WTN;  // output columns per wave
  constexpr int FNC = DUAL ? FN / 2 : FN;
  constexpr int OSZ = (MODE == WGRAD) ? (int)sizeof(OutT) : 2;
  constexpr int SSTRIDE = WTNC * OSZ + 16;  // bytes per strip row (16 bytes of padding)
  constexpr int SBYTES = 32 * SSTRIDE;
  constexpr int NSTRIP = (MODE == GATEUP) ? (BLK ? 1 : 3) : (MODE == DGRAD_DOWN ? 2 : 1);
  constexpr int CPRO = WTNC * OSZ / 16;  // 16-byte chunks per strip row
  constexpr int RPI = 64 / CPRO;         // rows covered by one wave-wide 16-byte access
  static_assert(64 % CPRO == 0 && 32 % RPI == 0, "strip shape");
  // Where they fit, the strips take the second LDS stage only (half of the waves in its A
  // part, half in its B part): the first stage is then free to receive the next tile's first
  // k-tile while the results are still being written out.
  // (the SwiGLU-backward epilogue needs the staging registers' room for its g/u rows: it sends
  // the request during its last strip, when that room is free, and stages nothing -- moving the
  // k-tile on into LDS at the end of that epilogue was measured 3 % slower)
  constexpr bool EARLY_REQUEST = (MODE != DGRAD_DOWN);
  constexpr int HALF_WAVES = Cfg::WM * Cfg::WN / 2;
  constexpr bool STAGE_EARLY = EARLY_REQUEST &&
                               NSTRIP * SBYTES * HALF_WAVES <= StA::LDS_ELEMS * 2 &&
                               NSTRIP * SBYTES * HALF_WAVES <= StB::LDS_ELEMS * 2;
  static_assert(NSTRIP * SBYTES * Cfg::WM * Cfg::WN <= lds_bytes<MODE, Cfg>(), "strips fit in the stages");
  char* strip = STAGE_EARLY
                    ? reinterpret_cast<char*>(wv < HALF_WAVES ? sA + StA::LDS_ELEMS : sB + StB::LDS_ELEMS) +
                          (wv % HALF_WAVES) * (NSTRIP * SBYTES)
                    : reinterpret_cast<char*>(smem) + wv * (NSTRIP * SBYTES);
  const int ldc = p.ld_c ? p.ld_c : p.N;  // outputs
  const int ldx = p.N;                    // epilogue inputs (g, u)
  // The accumulators of a strip are cleared for the next tile as soon as they are in LDS: the
  // moves fill the waits of the strip's LDS and global traffic instead of a slot before the
  // next main loop.
  auto zero_row = [&](int i) {
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  };
  // Blocked g/u (BLK): record of the 32 x 32 block (row block rb of row-tile slot `slot`, column
  // block cb = column / 32), GU_BLOCK_BYTES each: [g: q0q1 of lanes 0..63 | g: q2q3 | u: q0q1 |
  // u: q2q3], 16 bytes per lane and part, where lane l of the wave that owns the block holds row
  // l % 32 and columns 8*q + 4*(l/32) .. +3 of it for q = 0..3 (the accumulator layout above).
  // A wave-wide 16-byte access to one part covers 1 KB of consecutive addresses.  Row tiles are
  // numbered as the tile list numbers them (expert by expert, BM rows each), so that the forward
  // and the backward kernel agree on `slot` from the offsets alone.
  constexpr int GU_BLOCK_BYTES = 4096;
  const int n_cb = (p.N + 31) / 32;
  auto gu_block = [&](const void* base, const Tile& t, int rb, int cb, int ln) {
    return (char*)base + (((long long)t.slot * (BM / 32) + rb) * n_cb + cb) * GU_BLOCK_BYTES + ln * 16;
  };
  // `halfway` runs once, after the second of the FM strips; `last_rows_in` once the SwiGLU-backward
  // epilogue has taken the last g/u rows out of their registers
  auto epilogue = [&](const Tile& t, auto&& halfway, auto&& last_rows_in) {
    // Every per-lane address of the epilogue is derived from this copy of the lane index, which
    // the empty asm makes opaque: the compiler then recomputes them here, a handful of integer
    // operations per tile, instead of hoisting them out of the tile loop and holding a dozen
    // registers through the main loop for them.
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int l32 = lane_e & 31, lh = lane_e >> 5;
    const int row_in_pass = lane_e / CPRO, chunk_in_row = lane_e % CPRO;
    auto acc_ptr = [&](int plane, int j, int q) {  // 4 consecutive columns in accumulator layout
      return strip + plane * SBYTES + l32 * SSTRIDE + (j * 32 + 8 * q + 4 * lh) * OSZ;
    };
    auto put4 = [&](int plane, int j, int q, float a, float b, float c, float d) {
      if constexpr (OSZ == 4) *reinterpret_cast<f32x4*>(acc_ptr(plane, j, q)) = f32x4{a, b, c, d};
      else *reinterpret_cast<u32x2*>(acc_ptr(plane, j, q)) = u32x2{pack_bf16x2(a, b), pack_bf16x2(c, d)};
    };
    const int col_w0 = t.n0 + wn * WTNC;  // first output column of the wave
    char* C0 = (char*)p.C0;
    int m_shift = 0;  // WGRAD with two results: the rows of the second one start at m_split
    int m_lim = p.M;
    if constexpr (MODE == WGRAD) {
      if (p.m_split > 0) {
        if (t.m0 >= p.m_split) {
          C0 = (char*)p.C1 + (long long)t.e * (p.M - p.m_split) * p.N * OSZ;
          m_shift = p.m_split;
        } else {
          C0 += (long long)t.e * p.m_split * p.N * OSZ;
          m_lim = p.m_split;
        }
      } else {
        C0 += (long long)t.e * p.M * p.N * OSZ;
      }
    }
    const int row_lim = (MODE == WGRAD) ? m_lim : t.row_end;
    // row-wise pass over a strip: lane handles chunk (lane % CPRO) of row it*RPI + lane/CPRO
    auto store_rows = [&](int plane, int i, char* gbase /* element (0,0) of the output */) {
      const int rbase = (MODE == WGRAD ? t.m0 : t.row0) + wm * WTM + i * 32;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int rr = it * RPI + row_in_pass, ch = chunk_in_row;
        const u32x4 v = *reinterpret_cast<const u32x4*>(strip + plane * SBYTES + rr * SSTRIDE + ch * 16);
        const int r = rbase + rr, c = col_w0 + ch * (16 / OSZ);
        if (r < row_lim && c < p.N) {
          u32x4* dst = reinterpret_cast<u32x4*>(gbase + ((long long)(r - m_shift) * ldc + c) * OSZ);
          if (MODE == WGRAD && p.accumulate) {
            const u32x4 o = *dst;
            if constexpr (OSZ == 4) {
              const f32x4 sum = __builtin_bit_cast(f32x4, v) + __builtin_bit_cast(f32x4, o);
              *dst = __builtin_bit_cast(u32x4, sum);
            } else {
              *dst = u32x4{pack_bf16x2(bf16lo(v[0]) + bf16lo(o[0]), bf16hi(v[0]) + bf16hi(o[0])),
                           pack_bf16x2(bf16lo(v[1]) + bf16lo(o[1]), bf16hi(v[1]) + bf16hi(o[1])),
                           pack_bf16x2(bf16lo(v[2]) + bf16lo(o[2]), bf16hi(v[2]) + bf16hi(o[2])),
                           pack_bf16x2(bf16lo(v[3]) + bf16lo(o[3]), bf16hi(v[3]) + bf16hi(o[3]))};
            }
          } else {
            *dst = v;
          }
        }
      }
    };
    // DGRAD_DOWN reads g and u in the accumulator layout too: their rows come in as whole
    // 128-byte lines into registers (requested one strip ahead), pass through the strip and
    // are overwritten in place by dg and du.
    struct RowRegs {
      u32x4 g[32 / RPI], u[32 / RPI];
    };
    auto request_rows = [&](int i, RowRegs& rr_) {
      const int rbase = t.row0 + wm * WTM + i * 32;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int rr = it * RPI + row_in_pass, ch = chunk_in_row;
        const int r = rbase + rr, c = col_w0 + ch * (16 / OSZ);
        rr_.g[it] = u32x4{0, 0, 0, 0};
        rr_.u[it] = u32x4{0, 0, 0, 0};
        if (r < row_lim && c < p.N) {
          rr_.g[it] = *reinterpret_cast<const u32x4*>((const char*)p.X0 + ((long long)r * ldx + c) * OSZ);
          rr_.u[it] = *reinterpret_cast<const u32x4*>((const char*)p.X1 + ((long long)r * ldx + c) * OSZ);
        }
      }
    };
    auto rows_to_strip = [&](const RowRegs& rr_) {
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const int rr = it * RPI + row_in_pass, ch = chunk_in_row;
        *reinterpret_cast<u32x4*>(strip + 0 * SBYTES + rr * SSTRIDE + ch * 16) = rr_.g[it];
        *reinterpret_cast<u32x4*>(strip + 1 * SBYTES + rr * SSTRIDE + ch * 16) = rr_.u[it];
      }
    };
    // (BLK) the two 16-byte parts of g and of u for each of the strip's column blocks
    struct BlkRegs {
      u32x4 g[FNC][2], u[FNC][2];
    };
    auto request_block = [&](int i, int j, BlkRegs& b) {
      const int cb = (col_w0 + j * 32) / 32;
      const u32x4 zero = u32x4{0, 0, 0, 0};
      b.g[j][0] = b.g[j][1] = b.u[j][0] = b.u[j][1] = zero;
      if (t.row0 + wm * WTM + i * 32 < t.row_end && cb < n_cb) {
        const u32x4* rec = reinterpret_cast<const u32x4*>(gu_block(p.X0, t, wm * FM + i, cb, lane_e));
        // (read exactly once: streamed past the L2 lines the operand panels live in)
        b.g[j][0] = __builtin_nontemporal_load(rec + 0);
        b.g[j][1] = __builtin_nontemporal_load(rec + 64);
        b.u[j][0] = __builtin_nontemporal_load(rec + 128);
        b.u[j][1] = __builtin_nontemporal_load(rec + 192);
      }
    };
    RowRegs rows_in;
    BlkRegs blk_in;
    if constexpr (MODE == DGRAD_DOWN && BLK) {
#pragma unroll
      for (int j = 0; j < FNC; ++j) request_block(0, j, blk_in);
    } else if constexpr (MODE == DGRAD_DOWN) {
      request_rows(0, rows_in);
    }
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if constexpr (MODE == GATEUP) {
        // (BLK) blocks of a strip that starts past the end of the expert's rows are never read
        const bool strip_live = t.row0 + wm * WTM + i * 32 < t.row_end;
#pragma unroll
        for (int j = 0; j < FNC; ++j) {
          u32x2 gq[2], uq[2];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float g[4], u[4], a[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
              g[x] = acc[i][j][4 * q + x];
              u[x] = acc[i][j + FNC][4 * q + x];
              a[x] = g[x] * sigmoidf_(g[x]) * u[x];
            }
            put4(0, j, q, a[0], a[1], a[2], a[3]);
            if constexpr (BLK) {
              gq[q & 1] = u32x2{pack_bf16x2(g[0], g[1]), pack_bf16x2(g[2], g[3])};
              uq[q & 1] = u32x2{pack_bf16x2(u[0], u[1]), pack_bf16x2(u[2], u[3])};
              if (q & 1) {  // a 16-byte part of the record is complete: it leaves at once
                const int cb = (col_w0 + j * 32) / 32;
                if (p.C0 && strip_live && cb < n_cb) {
                  u32x4* rec = reinterpret_cast<u32x4*>(gu_block(p.C0, t, wm * FM + i, cb, lane_e));
                  // (written once, read by the backward pass much later: streaming stores)
                  __builtin_nontemporal_store(u32x4{gq[0][0], gq[0][1], gq[1][0], gq[1][1]}, rec + 64 * (q >> 1));
                  __builtin_nontemporal_store(u32x4{uq[0][0], uq[0][1], uq[1][0], uq[1][1]},
                                              rec + 128 + 64 * (q >> 1));
                }
              }
            } else if (p.C0) {
              put4(1, j, q, g[0], g[1], g[2], g[3]);
              put4(2, j, q, u[0], u[1], u[2], u[3]);
            }
          }
        }
        zero_row(i);
        store_rows(0, i, (char*)p.C2);
        if constexpr (!BLK) {
          if (p.C0) {
            store_rows(1, i, (char*)p.C0);
            store_rows(2, i, (char*)p.C1);
          }
        }
      } else if constexpr (MODE == DGRAD_DOWN && BLK) {
        // g and u arrive in the accumulator layout: nothing to rearrange.  The registers of column
        // block j are asked for the next strip's block as soon as this strip's block is computed.
        float rowdot = 0.f;
#pragma unroll
        for (int j = 0; j < FNC; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const u32x4 gv = blk_in.g[j][q >> 1], uv = blk_in.u[j][q >> 1];
            const uint32_t g01 = gv[2 * (q & 1)], g23 = gv[2 * (q & 1) + 1];
            const uint32_t u01 = uv[2 * (q & 1)], u23 = uv[2 * (q & 1) + 1];
            const float g[4] = {bf16lo(g01), bf16hi(g01), bf16lo(g23), bf16hi(g23)};
            const float u[4] = {bf16lo(u01), bf16hi(u01), bf16lo(u23), bf16hi(u23)};
            float dg[4], du[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
              const float dact = acc[i][j][4 * q + x];
              const float sg = sigmoidf_(g[x]);
              const float gs = g[x] * sg;                     // silu(g)
              du[x] = dact * gs;
              dg[x] = (dact * u[x]) * (sg + (gs - gs * sg));  // silu'(g) = s + g*s*(1-s)
              rowdot += du[x] * u[x];                         // dact * act
            }
            put4(0, j, q, dg[0], dg[1], dg[2], dg[3]);
            put4(1, j, q, du[0], du[1], du[2], du[3]);
            // (the running sum is wanted here, not at the end of the strip: left alone the compiler
            // may defer its chain of additions and keep every du and u alive for it)
            asm volatile("" : "+v"(rowdot));
          }
          __builtin_amdgcn_sched_barrier(0);  // (the loads must not move up: their registers are in use)
          if (i + 1 < FM) request_block(i + 1, j, blk_in);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (i + 1 == FM) last_rows_in();
        {
          rowdot += __shfl_xor(rowdot, 32, MOE_WAVE);
          const int r = t.row0 + wm * WTM + i * 32 + l32;
          if (lh == 0 && r < row_lim && p.C2)
            reinterpret_cast<float*>(p.C2)[(long long)((t.n0 / BNC) * Cfg::WN + wn) * p.R + r] = rowdot;
        }
        zero_row(i);
        store_rows(0, i, (char*)p.C0);
        store_rows(1, i, (char*)p.C1);
      } else if constexpr (MODE == DGRAD_DOWN) {
        rows_to_strip(rows_in);
        if (i + 1 < FM) request_rows(i + 1, rows_in);
        else last_rows_in();
        float rowdot = 0.f;  // this lane's share of <dact[row,:], act[row,:]>
#pragma unroll
        for (int j = 0; j < FNC; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const u32x2 gw = *reinterpret_cast<const u32x2*>(acc_ptr(0, j, q));
            const u32x2 uw = *reinterpret_cast<const u32x2*>(acc_ptr(1, j, q));
            const float g[4] = {bf16lo(gw[0]), bf16hi(gw[0]), bf16lo(gw[1]), bf16hi(gw[1])};
            const float u[4] = {bf16lo(uw[0]), bf16hi(uw[0]), bf16lo(uw[1]), bf16hi(uw[1])};
            float dg[4], du[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
              const float dact = acc[i][j][4 * q + x];
              const float sg = sigmoidf_(g[x]);
              const float gs = g[x] * sg;                     // silu(g)
              du[x] = dact * gs;
              dg[x] = (dact * u[x]) * (sg + (gs - gs * sg));  // silu'(g) = s + g*s*(1-s)
              rowdot += du[x] * u[x];                         // dact * act
            }
            put4(0, j, q, dg[0], dg[1], dg[2], dg[3]);
            put4(1, j, q, du[0], du[1], du[2], du[3]);
            asm volatile("" : "+v"(rowdot));  // (summed here: see the blocked variant above)
          }
        {
          // One partial per 64-column block and row (block-major, so that a wave writes 32
          // consecutive floats): the row's sum over all blocks is
          // gate * <dy[token], y[row]>, i.e. what the gate's gradient needs, so that nobody
          // has to read y again.  Written, not accumulated: the caller adds the blocks up in
          // a fixed order.
          rowdot += __shfl_xor(rowdot, 32, MOE_WAVE);
          const int r = t.row0 + wm * WTM + i * 32 + l32;
          if (lh == 0 && r < row_lim && p.C2)
            reinterpret_cast<float*>(p.C2)[(long long)((t.n0 / BNC) * Cfg::WN + wn) * p.R + r] = rowdot;
        }
        zero_row(i);
        store_rows(0, i, (char*)p.C0);
        store_rows(1, i, (char*)p.C1);
      } else {
#pragma unroll
        for (int j = 0; j < FNC; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            put4(0, j, q, acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
        zero_row(i);
        store_rows(0, i, C0);
      }
      if (i == (FM > 1 ? 1 : 0)) halfway();
    }
  };

  // ---- the tile loop
  // At the top of the loop the first k-tile of `cur` is already on its way into the staging
  // registers (requested before the previous tile's epilogue).
  auto request_first = [&](const Tile& t) {
    if (0 < t.nkt) {
      load_tile(t, 0, stg);
    } else {
      // (nothing will be read from the staging registers: say so, or they stay alive through the
      // epilogue on account of this path)
#pragma unroll
      for (int c = 0; c < NCH; ++c) asm volatile("" : "=v"(stg.v[c]));
    }
  };
  Tile cur;
  if (t_next >= t_hi || !locate(tile_at(t_next), cur)) return;
  request_first(cur);
  bool staged = false;  // k-tile 0 of `cur` already sits in LDS stage 0, k-tile 1 is on its way
#pragma unroll
  for (int i = 0; i < FM; ++i) zero_row(i);  // later tiles find them cleared by the epilogue
  for (;;) {
    // The last row tile of an expert is mostly short.  A wave whose rows all lie past its end
    // multiplies nothing: it only keeps moving operand chunks and meets the barriers (the
    // same ones in the same order as the waves that work), so that such a tile costs the
    // matrix pipe half of a full one.
    // The fragment registers carry nothing from one tile to the next.  The compiler cannot see that
    // (their first reads sit behind conditions it does not correlate with the loops that use them)
    // and would keep all of them alive through the epilogue; an empty asm that "writes" them ends
    // their live ranges here at no cost.
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < FM; ++i) asm volatile("" : "=v"(fr[h].a[i]));
#pragma unroll
      for (int j = 0; j < FN; ++j) asm volatile("" : "=v"(fr[h].b[j]));
    }
    const bool idle =
        (MODE != WGRAD) && __builtin_amdgcn_readfirstlane((int)(wm * WTM >= cur.row_end - cur.row0)) != 0;
    // where the next tile lies is worked out now (a binary search in LDS and some address
    // arithmetic), in the shadow of this tile's first MFMAs, not between the tiles
    Tile nxt;
    t_next += t_step ? t_step : 1;
    const bool more = t_next < t_hi && locate(tile_at(t_next), nxt);
    const int nkt = cur.nkt;
    if (nkt > 0) {
      if (!staged) {
        store_tile(stg, 0);
        if (1 < nkt) load_tile(cur, 1, stg);
        lds_barrier();
      }
      if (!idle) f_read_all(0, 0, fr[0]);
    }
    int kt = 0;
    if (idle) {
      for (; kt < nkt; ++kt) {
        const bool has1 = kt + 1 < nkt, has2 = kt + 2 < nkt;
        if (has1) {
          store_tile(stg, (kt & 1) ^ 1);
          if (has2) load_tile(cur, kt + 2, stg);
          lds_barrier();
        }
      }
    }
    // steady iterations (two at a time: the stage index is a compile-time constant): k-tile
    // kt+2 exists and nothing needs masking
    const int steady_end = cur.need_mask ? 0 : nkt - 2;
    for (; kt + 1 < steady_end; kt += 2) {
      body(integral_constant<int, 0>{}, cur, kt);
      body(integral_constant<int, 1>{}, cur, kt + 1);
    }
    for (; kt < nkt; ++kt) {  // last iterations (and every iteration when masking): same
      const int buf = kt & 1;  // order of events, conditions evaluated, no static schedule
      const bool has1 = kt + 1 < nkt, has2 = kt + 2 < nkt;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) f_read_all(buf, ks + 1, fr[(ks + 1) & 1]);
        if (ks == 0 && has1) {
          store_tile(stg, buf ^ 1);
          if (has2) load_tile(cur, kt + 2, stg);
        }
        if (ks == KS - 1 && has1) {
          lds_barrier();
          f_read_all(buf ^ 1, 0, fr[0]);
        }
        mma_all(fr[ks & 1]);
      }
    }
    // the next tile's first k-tiles travel while this tile's results are written out
    if (EARLY_REQUEST && more) request_first(nxt);
    lds_barrier();  // every wave is done reading the operand stages
    // Half-way through the epilogue the next tile's first k-tile has arrived: it moves on
    // into LDS stage 0 (idle: the strips live in stage 1) and its registers fetch the second
    // k-tile, so that the next main loop starts with both in place instead of waiting for
    // a load it has only just issued.
    staged = false;
    auto stage_next = [&]() {
      if constexpr (STAGE_EARLY) {
        if (more && nxt.nkt > 0) {
          store_tile(stg, 0);
          if (1 < nxt.nkt) load_tile(nxt, 1, stg);
          staged = true;
        }
      }
    };
    // Where the epilogue needs the staging registers' room for most of its length, the request
    // goes out as soon as that room is free: during the last of its strips.
    bool requested = EARLY_REQUEST;
    auto late_request = [&]() {
      if constexpr (!EARLY_REQUEST) {
        if (more) request_first(nxt);
        requested = true;
      }
    };
    if (idle) stage_next();
    else epilogue(cur, stage_next, late_request);
    if (!more) break;
    if (!requested) request_first(nxt);
    lds_barrier();  // every wave is done with its strip, and stage 0 is complete if staged
    cur = nxt;
  }
}

#ifndef MOE_BM
#define MOE_BM 256
#define MOE_BN 256
#define MOE_BK 64
#define MOE_WM 2
#define MOE_WN 4
#endif
using CfgMain = TileCfg<MOE_BM, MOE_BN, MOE_BK, MOE_WM, MOE_WN>;
// Row tiles of half the height (the eight waves 64 x 64 each) for launches too small to give even
// half of the compute units one of the large tiles: twice the tiles, each at about 0.7 of the
// large tile's cost, spread such a launch over twice the compute units.
using CfgSmall = TileCfg<MOE_BM / 2, MOE_BN, MOE_BK, MOE_WM, MOE_WN>;

int compute_units() {
  static int cus[MOE_MAX_DEVICES];  // per GPU; 0 = not asked yet
  const int dev = moe_current_device();
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev] = n;
  }
  return cus[dev];
}

// `ntiles` is the number of tile slots; the grid is as many workgroups as are resident at
// once (one or two per compute unit, by LDS footprint), or fewer when there are fewer tiles.
template <int MODE, typename Cfg, typename OutT, bool BLK = false>
int launch(const GemmArgs& a, long long ntiles, hipStream_t s) {
  if (ntiles <= 0) return 0;
  auto kern = grouped_gemm_kernel<MODE, Cfg, OutT, BLK>;
  constexpr int LDS = lds_bytes<MODE, Cfg>();
  static bool attr_done[MOE_MAX_DEVICES];  // per GPU and instantiation
  const int dev = moe_current_device();
  if (!attr_done[dev]) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (e != hipSuccess) return (int)e;
    attr_done[dev] = true;
  }
  // as many workgroups as can be resident at once: the LDS footprint decides how many share a CU
  const long long slots = (long long)compute_units() * ((160 * 1024) / LDS >= Cfg::WGS_PER_CU ? Cfg::WGS_PER_CU : 1);
  const unsigned grid = (unsigned)(ntiles < slots ? ntiles : slots);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::NT), LDS, s, a);
  return moe_launch_status();
}

int check_common(const int32_t* offs, int64_t E, int64_t R, int64_t H, int64_t I) {
  if (!offs) return MOE_ERR_NULL;
  if (E <= 0 || R < 0 || H <= 0 || I <= 0 || (H % 8) || (I % 8)) return MOE_ERR_SHAPE;
  if (E > GEMM_MAX_E || R > (int64_t)1 << 30 || H > (1 << 16) || I > (1 << 16)) return MOE_ERR_LIMIT;
  // Row and column positions are 64-bit wherever they are multiplied by a row length; what is
  // 32-bit is the per-lane offset inside one tile's window (at most 256 rows of 65536 elements)
  // and the tile index: rows / 256 + E row slots times the column tiles of the widest output.
  const int64_t widest = H > I ? H : I;
  if ((R / 256 + E + 1) * ((widest + 127) / 128) >= ((int64_t)1 << 31)) return MOE_ERR_LIMIT;
  return 0;
}

template <typename Cfg>
int row_slots(int64_t R, int64_t E) {
  return (int)((R + Cfg::BM - 1) / Cfg::BM + E);
}

// Which row-tile height a row-ragged launch uses: decided from the shapes alone (never from the
// routing: no host synchronisation), the same way for the forward kernel that writes blocked g/u
// and the backward kernel that reads it (both pass I as `cols`).  Measured on the two small
// benchmark configurations: 4096 rows of 8 experts (48 large tiles by this count) run 24 % faster
// on the small tiles, 16384 rows (144) no faster.  `forced_row_tile` (0: automatic) is a test hook.
int forced_row_tile = 0;
bool small_row_tiles(int64_t R, int64_t E, int64_t cols) {
  if (forced_row_tile) return forced_row_tile == CfgSmall::BM;
  const int64_t tiles = (int64_t)row_slots<CfgMain>(R, E) * ((cols + CfgMain::BN - 1) / CfgMain::BN);
  return 2 * tiles < (int64_t)compute_units();
}
template <typename F>
int with_row_tile(bool small, F&& f) {
  return small ? f(CfgSmall{}) : f(CfgMain{});
}

}  // namespace

extern "C" int moe_gemm_gateup_swiglu_fwd(const uint16_t* xp, const uint16_t* w1, const uint16_t* w3,
                                          const int32_t* offs, int64_t E, int64_t R, int64_t H,
                                          int64_t I, uint16_t* g, uint16_t* u, uint16_t* act,
                                          void* stream) {
  if (int rc = check_common(offs, E, R, H, I)) return rc;
  if (R == 0) return 0;
  MOE_CHECK_PTR(xp); MOE_CHECK_PTR(w1); MOE_CHECK_PTR(w3); MOE_CHECK_PTR(act);
  if ((g == nullptr) != (u == nullptr)) return MOE_ERR_NULL;
  return with_row_tile(small_row_tiles(R, E, I), [&](auto cfg) {
    using Cfg = decltype(cfg);
    GemmArgs a{};
    a.A0 = xp; a.B0 = w1; a.B1 = w3; a.C0 = g; a.C1 = u; a.C2 = act; a.offs = offs;
    a.E = (int)E; a.R = (int)R; a.N = (int)I; a.K = (int)H;
    a.n_tiles = (int)((I + Cfg::BN / 2 - 1) / (Cfg::BN / 2));
    a.m_slots = row_slots<Cfg>(R, E);
    return launch<GATEUP, Cfg, uint16_t>(a, (long long)a.n_tiles * a.m_slots, (hipStream_t)stream);
  });
}

// Bytes of the blocked g/u buffer: one 4 KB record per 32 x 32 block of every row-tile slot the
// tile list can have (ceil(R/256) + E bounds their number whatever the routing).
extern "C" int64_t moe_gu_blocked_bytes(int64_t R, int64_t E, int64_t I) {
  if (R <= 0 || E <= 0 || I <= 0) return 0;
  using Cfg = CfgMain;
  return (int64_t)row_slots<Cfg>(R, E) * (Cfg::BM / 32) * ((I + 31) / 32) * 4096;
}

extern "C" int moe_gemm_gateup_swiglu_fwd_blocked(const uint16_t* xp, const uint16_t* w1, const uint16_t* w3,
                                                  const int32_t* offs, int64_t E, int64_t R, int64_t H,
                                                  int64_t I, void* gu_blocked, uint16_t* act, void* stream) {
  if (int rc = check_common(offs, E, R, H, I)) return rc;
  if (R == 0) return 0;
  MOE_CHECK_PTR(xp); MOE_CHECK_PTR(w1); MOE_CHECK_PTR(w3); MOE_CHECK_PTR(act); MOE_CHECK_PTR(gu_blocked);
  return with_row_tile(small_row_tiles(R, E, I), [&](auto cfg) {
    using Cfg = decltype(cfg);
    GemmArgs a{};
    a.A0 = xp; a.B0 = w1; a.B1 = w3; a.C0 = gu_blocked; a.C2 = act; a.offs = offs;
    a.E = (int)E; a.R = (int)R; a.N = (int)I; a.K = (int)H;
    a.n_tiles = (int)((I + Cfg::BN / 2 - 1) / (Cfg::BN / 2));
    a.m_slots = row_slots<Cfg>(R, E);
    return launch<GATEUP, Cfg, uint16_t, true>(a, (long long)a.n_tiles * a.m_slots, (hipStream_t)stream);
  });
}

extern "C" int moe_gemm_down_fwd(const uint16_t* act, const uint16_t* w2, const int32_t* offs,
                                 int64_t E, int64_t R, int64_t H, int64_t I, uint16_t* y,
                                 void* stream) {
  if (int rc = check_common(offs, E, R, H, I)) return rc;
  if (R == 0) return 0;
  MOE_CHECK_PTR(act); MOE_CHECK_PTR(w2); MOE_CHECK_PTR(y);
  return with_row_tile(small_row_tiles(R, E, H), [&](auto cfg) {
    using Cfg = decltype(cfg);
    GemmArgs a{};
    a.A0 = act; a.B0 = w2; a.C0 = y; a.offs = offs;
    a.E = (int)E; a.R = (int)R; a.N = (int)H; a.K = (int)I;
    a.n_tiles = (int)((H + Cfg::BN - 1) / Cfg::BN);
    a.m_slots = row_slots<Cfg>(R, E);
    return launch<DOWN, Cfg, uint16_t>(a, (long long)a.n_tiles * a.m_slots, (hipStream_t)stream);
  });
}

// Test hook: 0 lets every row-ragged launch choose its row-tile height (the default), 128 or 256
// forces it.  Process-wide and not synchronised: for tests that want every shape on every tile
// configuration, not for production callers.  Returns the previous setting.
extern "C" int moe_gemm_force_row_tile(int rows) {
  const int before = forced_row_tile;
  if (rows == 0 || rows == CfgSmall::BM || rows == CfgMain::BM) forced_row_tile = rows;
  return before;
}

extern "C" int64_t moe_dgate_blocks(int64_t I) {
  using Cfg = CfgMain;
  return I <= 0 ? 0 : ((I + Cfg::BN - 1) / Cfg::BN) * Cfg::WN;
}

static int dgrad_down_impl(const uint16_t* dyp, const uint16_t* w2, const uint16_t* g, const uint16_t* u,
                           const int32_t* offs, int64_t E, int64_t R, int64_t H, int64_t I,
                           uint16_t* dg, uint16_t* du, float* dgate_part, void* stream, int64_t ld_out = 0) {
  if (int rc = check_common(offs, E, R, H, I)) return rc;
  if (R == 0) return 0;
  MOE_CHECK_PTR(dyp); MOE_CHECK_PTR(w2); MOE_CHECK_PTR(g); MOE_CHECK_PTR(u);
  MOE_CHECK_PTR(dg); MOE_CHECK_PTR(du);
  return with_row_tile(small_row_tiles(R, E, I), [&](auto cfg) {
    using Cfg = decltype(cfg);
    GemmArgs a{};
    a.C2 = dgate_part;
    a.A0 = dyp; a.B0 = w2; a.X0 = g; a.X1 = u; a.C0 = dg; a.C1 = du; a.offs = offs;
    a.E = (int)E; a.R = (int)R; a.N = (int)I; a.K = (int)H; a.ld_c = (int)ld_out;
    a.n_tiles = (int)((I + Cfg::BN - 1) / Cfg::BN);
    a.m_slots = row_slots<Cfg>(R, E);
    return launch<DGRAD_DOWN, Cfg, uint16_t>(a, (long long)a.n_tiles * a.m_slots, (hipStream_t)stream);
  });
}

extern "C" int moe_gemm_dgrad_down_swiglu_bwd(const uint16_t* dyp, const uint16_t* w2,
                                              const uint16_t* g, const uint16_t* u,
                                              const int32_t* offs, int64_t E, int64_t R, int64_t H,
                                              int64_t I, uint16_t* dg, uint16_t* du, void* stream) {
  return dgrad_down_impl(dyp, w2, g, u, offs, E, R, H, I, dg, du, nullptr, stream);
}

extern "C" int moe_gemm_dgrad_down_swiglu_bwd_dgate(const uint16_t* dyp, const uint16_t* w2,
                                                    const uint16_t* g, const uint16_t* u,
                                                    const int32_t* offs, int64_t E, int64_t R,
                                                    int64_t H, int64_t I, uint16_t* dg, uint16_t* du,
                                                    float* dgate_part, void* stream) {
  if (R > 0 && !dgate_part) return MOE_ERR_NULL;
  return dgrad_down_impl(dyp, w2, g, u, offs, E, R, H, I, dg, du, dgate_part, stream);
}

extern "C" int moe_gemm_dgrad_down_swiglu_bwd_blocked(const uint16_t* dyp, const uint16_t* w2,
                                                      const void* gu_blocked, const int32_t* offs, int64_t E,
                                                      int64_t R, int64_t H, int64_t I, uint16_t* dg,
                                                      uint16_t* du, int64_t ld_out, float* dgate_part,
                                                      void* stream) {
  if (int rc = check_common(offs, E, R, H, I)) return rc;
  if (R == 0) return 0;
  MOE_CHECK_PTR(dyp); MOE_CHECK_PTR(w2); MOE_CHECK_PTR(gu_blocked); MOE_CHECK_PTR(dg); MOE_CHECK_PTR(du);
  if (ld_out != 0 && (ld_out < I || (ld_out % 8) != 0 || ld_out > (1 << 17))) return MOE_ERR_SHAPE;
  return with_row_tile(small_row_tiles(R, E, I), [&](auto cfg) {
    using Cfg = decltype(cfg);
    GemmArgs a{};
    a.C2 = dgate_part;
    a.A0 = dyp; a.B0 = w2; a.X0 = (const uint16_t*)gu_blocked; a.C0 = dg; a.C1 = du; a.offs = offs;
    a.E = (int)E; a.R = (int)R; a.N = (int)I; a.K = (int)H; a.ld_c = (int)ld_out;
    a.n_tiles = (int)((I + Cfg::BN - 1) / Cfg::BN);
    a.m_slots = row_slots<Cfg>(R, E);
    return launch<DGRAD_DOWN, Cfg, uint16_t, true>(a, (long long)a.n_tiles * a.m_slots, (hipStream_t)stream);
  });
}

// The two row gradients side by side in one buffer: dgu [R, 2I], row = [dg row | du row].  The
// weight gradients of the gate and up stacks then are ONE grouped product, dgu^T * xp, whose
// result rows 0..I-1 are dW1 and I..2I-1 dW3 (moe_gemm_wgrad_pair).
extern "C" int moe_gemm_dgrad_down_swiglu_bwd_packed(const uint16_t* dyp, const uint16_t* w2,
                                                     const uint16_t* g, const uint16_t* u,
                                                     const int32_t* offs, int64_t E, int64_t R,
                                                     int64_t H, int64_t I, uint16_t* dgu,
                                                     float* dgate_part, void* stream) {
  if (R > 0 && !dgu) return MOE_ERR_NULL;
  return dgrad_down_impl(dyp, w2, g, u, offs, E, R, H, I, dgu, dgu ? dgu + I : nullptr, dgate_part, stream, 2 * I);
}

static int dgrad_gateup_impl(const uint16_t* dg, const uint16_t* du, int64_t ld_in, const uint16_t* w1,
                             const uint16_t* w3, const int32_t* offs, int64_t E, int64_t R, int64_t H,
                             int64_t I, uint16_t* dxp, void* stream) {
  if (int rc = check_common(offs, E, R, H, I)) return rc;
  if (R == 0) return 0;
  MOE_CHECK_PTR(dg); MOE_CHECK_PTR(du); MOE_CHECK_PTR(w1); MOE_CHECK_PTR(w3); MOE_CHECK_PTR(dxp);
  return with_row_tile(small_row_tiles(R, E, H), [&](auto cfg) {
    using Cfg = decltype(cfg);
    GemmArgs a{};
    a.A0 = dg; a.A1 = du; a.B0 = w1; a.B1 = w3; a.C0 = dxp; a.offs = offs; a.ld_a = (int)ld_in;
    a.E = (int)E; a.R = (int)R; a.N = (int)H; a.K = (int)I;
    a.n_tiles = (int)((H + Cfg::BN - 1) / Cfg::BN);
    a.m_slots = row_slots<Cfg>(R, E);
    return launch<DGRAD_GATEUP, Cfg, uint16_t>(a, (long long)a.n_tiles * a.m_slots, (hipStream_t)stream);
  });
}

extern "C" int moe_gemm_dgrad_gateup_packed(const uint16_t* dgu, const uint16_t* w1, const uint16_t* w3,
                                            const int32_t* offs, int64_t E, int64_t R, int64_t H,
                                            int64_t I, uint16_t* dxp, void* stream) {
  if (R > 0 && !dgu) return MOE_ERR_NULL;
  return dgrad_gateup_impl(dgu, dgu ? dgu + I : nullptr, 2 * I, w1, w3, offs, E, R, H, I, dxp, stream);
}

extern "C" int moe_gemm_wgrad_pair(const uint16_t* dgu, const uint16_t* xp, const int32_t* offs, int64_t E,
                                   int64_t R, int64_t I, int64_t H, void* dw1, void* dw3, int dw_dtype,
                                   int accumulate, void* stream) {
  if (int rc = check_common(offs, E, R, I, H)) return rc;  // (the stacked result has 2*I <= 131072 rows)
  // a 256-row tile of the stacked result must not straddle the two halves
  if ((I % CfgMain::BM) != 0) return MOE_ERR_SHAPE;
  MOE_CHECK_PTR(dw1); MOE_CHECK_PTR(dw3);
  if (R > 0) { MOE_CHECK_PTR(dgu); MOE_CHECK_PTR(xp); }
  if (dw_dtype != MOE_DT_BF16 && dw_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  using Cfg = CfgMain;
  GemmArgs a{};
  a.A0 = dgu; a.B0 = xp; a.C0 = dw1; a.C1 = dw3; a.offs = offs; a.m_split = (int)I;
  a.E = (int)E; a.R = (int)R; a.M = (int)(2 * I); a.N = (int)H; a.accumulate = accumulate;
  a.n_tiles = (int)((H + Cfg::BN - 1) / Cfg::BN);
  a.m_slots = (int)((2 * I + Cfg::BM - 1) / Cfg::BM);
  const long long nblocks = (long long)a.n_tiles * a.m_slots * E;
  if (dw_dtype == MOE_DT_F32) return launch<WGRAD, Cfg, float>(a, nblocks, (hipStream_t)stream);
  return launch<WGRAD, Cfg, uint16_t>(a, nblocks, (hipStream_t)stream);
}

extern "C" int moe_gemm_dgrad_gateup(const uint16_t* dg, const uint16_t* du, const uint16_t* w1,
                                     const uint16_t* w3, const int32_t* offs, int64_t E, int64_t R,
                                     int64_t H, int64_t I, uint16_t* dxp, void* stream) {
  return dgrad_gateup_impl(dg, du, 0, w1, w3, offs, E, R, H, I, dxp, stream);
}

extern "C" int moe_gemm_wgrad(const uint16_t* a_, const uint16_t* b_, const int32_t* offs, int64_t E,
                              int64_t R, int64_t M, int64_t N, void* dw, int dw_dtype,
                              int accumulate, void* stream) {
  if (int rc = check_common(offs, E, R, M, N)) return rc;
  MOE_CHECK_PTR(dw);
  if (R > 0) { MOE_CHECK_PTR(a_); MOE_CHECK_PTR(b_); }
  if (dw_dtype != MOE_DT_BF16 && dw_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  using Cfg = CfgMain;
  GemmArgs a{};
  a.A0 = a_; a.B0 = b_; a.C0 = dw; a.offs = offs;
  a.E = (int)E; a.R = (int)R; a.M = (int)M; a.N = (int)N; a.accumulate = accumulate;
  a.n_tiles = (int)((N + Cfg::BN - 1) / Cfg::BN);
  a.m_slots = (int)((M + Cfg::BM - 1) / Cfg::BM);
  const long long nblocks = (long long)a.n_tiles * a.m_slots * E;
  if (dw_dtype == MOE_DT_F32)
    return launch<WGRAD, Cfg, float>(a, nblocks, (hipStream_t)stream);
  return launch<WGRAD, Cfg, uint16_t>(a, nblocks, (hipStream_t)stream);
}
