// Lock-step CPU emulation of one workgroup of the small-input dispatch kernel: one OS thread per
// lane, wave intrinsics (shuffles, ballots, barriers) through std::barrier, every global access
// bounds-checked.  The kernel's text is spliced in from csrc/dispatch.hip by the test that builds
// this file (marker KERNEL_SOURCE below), so what runs here is the product's own code.  A wave
// intrinsic reached by only some lanes of a wave (undefined on the GPU: the inactive lanes' values
// are read) shows up here as a deadlock, an out-of-bounds index as an abort.
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <vector>
#include <thread>
#include <barrier>
#include <atomic>
#include <cassert>
#include <algorithm>
#include <numeric>
#define MOE_WAVE 64
constexpr int ROWS_PER_WAVE = 256;
constexpr int SMALL_WAVES = 16;
constexpr int NT = SMALL_WAVES * MOE_WAVE;
struct Dim { int x; };
thread_local Dim threadIdx; static Dim blockDim{NT};
static int g_lds_words = 0; static int* g_lds = nullptr;
static std::barrier<>* g_block; static std::barrier<>* g_wave[SMALL_WAVES];
static long long g_slot[SMALL_WAVES][MOE_WAVE];
template <typename T> struct Checked { T* p; long long n; const char* name;
  T& operator[](long long i) const { if (i < 0 || i >= n) { fprintf(stderr, "OOB %s[%lld] of %lld (thread %d)\n", name, i, n, threadIdx.x); abort(); } return p[i]; } };
struct LdsPtr;  // LDS accesses are checked through g_lds bounds below
static inline int lane_id() { return threadIdx.x & 63; }
static inline int wv_() { return threadIdx.x >> 6; }
static inline void __syncthreads() { g_block->arrive_and_wait(); }
static inline void __builtin_amdgcn_wave_barrier() { g_wave[wv_()]->arrive_and_wait(); }
static inline long long xchg(long long v, int src) { g_slot[wv_()][lane_id()] = v; g_wave[wv_()]->arrive_and_wait(); long long r = g_slot[wv_()][src & 63]; g_wave[wv_()]->arrive_and_wait(); return r; }
static inline int __shfl_up(int v, int off, int) { int l = lane_id(); long long r = xchg(v, l - off < 0 ? l : l - off); return (int)r; }
static inline int __shfl_xor(int v, int m, int) { return (int)xchg(v, lane_id() ^ m); }
static inline int __shfl(int v, int src, int) { return (int)xchg(v, src); }
static inline unsigned long long __ballot(bool p) { g_slot[wv_()][lane_id()] = p; g_wave[wv_()]->arrive_and_wait(); unsigned long long m = 0; for (int i = 0; i < 64; ++i) if (g_slot[wv_()][i]) m |= 1ull << i; g_wave[wv_()]->arrive_and_wait(); return m; }
static inline int __popcll(unsigned long long v) { return __builtin_popcountll(v); }
static inline int atomicAdd(int* p, int v) { if (p < g_lds || p >= g_lds + g_lds_words) { fprintf(stderr, "OOB LDS atomic\n"); abort(); } return __atomic_fetch_add(p, v, __ATOMIC_SEQ_CST); }
static inline int wave_incl_scan(int v) { const int lane = lane_id(); for (int off = 1; off < MOE_WAVE; off <<= 1) { int o = __shfl_up(v, off, MOE_WAVE); if (lane >= off) v += o; } return v; }
static inline int clamp_expert(int e, int E) { return e < 0 ? 0 : (e >= E ? E - 1 : e); }
// KERNEL_SOURCE
int main() {
  for (int w = 0; w < SMALL_WAVES; ++w) g_wave[w] = new std::barrier<>(MOE_WAVE);
  g_block = new std::barrier<>(NT);
  struct Case { int R, E; };
  srand(1);
  for (Case c : {Case{512, 8}, Case{300, 9}, Case{1, 1}, Case{777, 3}, Case{1500, 64}, Case{700, 512}}) {
    int R = c.R, E = c.E, NW = (R + ROWS_PER_WAVE - 1) / ROWS_PER_WAVE;
    std::vector<int32_t> ids(R), counts(E, -7), offs(E + 1, -7), p2r(R, -7), r2p(R, -7); int32_t bad = -7;
    for (auto& v : ids) v = rand() % E;
    if (R > 100) { ids[5] = E + 3; ids[77] = -2; }
    g_lds_words = NW * E + E + 1; std::vector<int> lds(g_lds_words, 0x7fffffff); g_lds = lds.data();
    std::vector<std::thread> th;
    for (int t = 0; t < NT; ++t) th.emplace_back([&, t] { threadIdx.x = t;
      dispatch_small_kernel(Checked<const int32_t>{ids.data(), R, "ids"}, R, E, NW, Checked<int32_t>{counts.data(), E, "counts"}, Checked<int32_t>{offs.data(), E + 1, "offs"}, Checked<int32_t>{p2r.data(), R, "pos_to_row"}, Checked<int32_t>{r2p.data(), R, "row_to_pos"}, &bad); });
    for (auto& t : th) t.join();
    // reference
    std::vector<int> cl(R); for (int i = 0; i < R; ++i) cl[i] = clamp_expert(ids[i], E);
    std::vector<int> order(R); std::iota(order.begin(), order.end(), 0); std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return cl[a] < cl[b]; });
    bool ok = true; for (int i = 0; i < R; ++i) ok &= (p2r[i] == order[i]) && (r2p[order[i]] == i);
    int nb = 0; for (int i = 0; i < R; ++i) nb += ids[i] < 0 || ids[i] >= E;
    ok &= bad == nb; ok &= offs[E] == R;
    printf("R=%d E=%d %s\n", R, E, ok ? "ok" : "MISMATCH"); fflush(stdout);
    if (!ok) return 1;
  }
}
