// The whole forward pass of the layer body behind one call: routing, dispatch, row gather, the two
// grouped GEMMs and the combine (model/modules/mlp.py:101-167) enqueued back to back on the
// caller's stream, with every intermediate in a workspace the caller provides.  For callers that
// only want the output (inference, evaluation, a forward under no_grad): one crossing of the FFI
// boundary and two buffers instead of six crossings and a dozen.  Nothing here touches the GPU
// itself: the kernels are the ones the separate entry points launch, in the same order, so the
// output holds the same bits.
#include "common.h"

namespace {

constexpr int64_t ALIGN = 256;
int64_t up(int64_t n) { return (n + ALIGN - 1) / ALIGN * ALIGN; }

struct Carve {
  int64_t ids, gates, counts, offs, pos_to_row, row_to_pos, xp, act, y, dispatch, total;
};

Carve carve(int64_t T, int64_t H, int64_t E, int64_t I, int64_t k) {
  const int64_t R = T * k;
  Carve c;
  int64_t at = 0;
  auto take = [&](int64_t bytes) {
    const int64_t here = at;
    at += up(bytes > 0 ? bytes : 1);
    return here;
  };
  c.ids = take(R * 4);
  c.gates = take(R * 4);
  c.counts = take(E * 4);
  c.offs = take((E + 1) * 4);
  c.pos_to_row = take(R * 4);
  c.row_to_pos = take(R * 4);
  c.xp = take(R * H * 2);
  c.act = take(R * I * 2);
  c.y = take(R * H * 2);
  c.dispatch = take(moe_dispatch_workspace_bytes(R, E));
  c.total = at;
  return c;
}

bool sizes_ok(int64_t T, int64_t H, int64_t E, int64_t I, int64_t k) {
  return T >= 0 && H > 0 && E > 0 && I > 0 && k > 0 && k <= MOE_MAX_TOPK && k <= E && E <= MOE_MAX_EXPERTS &&
         H <= 65536 && I <= 65536 && T <= ((int64_t)1 << 30) / k;
}

}  // namespace

extern "C" int64_t moe_ffn_forward_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t I, int64_t k) {
  if (!sizes_ok(T, H, E, I, k)) return 0;
  return carve(T, H, E, I, k).total;
}

extern "C" int moe_ffn_forward(const void* x, int x_dtype, const void* logits, int logits_dtype,
                               const float* bias, const uint16_t* w1, const uint16_t* w3, const uint16_t* w2,
                               int64_t T, int64_t H, int64_t E, int64_t I, int64_t k, void* out,
                               int out_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  if (T < 0 || H <= 0 || E <= 0 || I <= 0 || k <= 0 || H % 8 != 0 || I % 8 != 0) return MOE_ERR_SHAPE;
  if (!sizes_ok(T, H, E, I, k)) return MOE_ERR_LIMIT;
  if (x_dtype != MOE_DT_BF16 && x_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  if (logits_dtype != MOE_DT_BF16 && logits_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  if (out_dtype != MOE_DT_BF16 && out_dtype != MOE_DT_F32) return MOE_ERR_DTYPE;
  if (T == 0) return 0;
  MOE_CHECK_PTR(x);
  MOE_CHECK_PTR(logits);
  MOE_CHECK_PTR(w1);
  MOE_CHECK_PTR(w3);
  MOE_CHECK_PTR(w2);
  MOE_CHECK_PTR(out);
  MOE_CHECK_PTR(workspace);
  const Carve c = carve(T, H, E, I, k);
  if (workspace_bytes < c.total) return MOE_ERR_WORKSPACE;
  char* ws = (char*)workspace;
  const int64_t R = T * k;
  int32_t* ids = (int32_t*)(ws + c.ids);
  float* gates = (float*)(ws + c.gates);
  int32_t* counts = (int32_t*)(ws + c.counts);
  int32_t* offs = (int32_t*)(ws + c.offs);
  int32_t* pos_to_row = (int32_t*)(ws + c.pos_to_row);
  int32_t* row_to_pos = (int32_t*)(ws + c.row_to_pos);
  uint16_t* xp = (uint16_t*)(ws + c.xp);
  uint16_t* act = (uint16_t*)(ws + c.act);
  uint16_t* y = (uint16_t*)(ws + c.y);
  int rc = moe_router_topk_fwd(logits, logits_dtype, bias, T, E, k, ids, gates, stream);
  if (rc) return rc;
  rc = moe_histogram_scan(ids, R, E, counts, offs, pos_to_row, row_to_pos, ws + c.dispatch,
                          moe_dispatch_workspace_bytes(R, E), stream);
  if (rc) return rc;
  rc = k > 1 ? moe_permute_fwd_scatter(x, x_dtype, row_to_pos, T, H, k, xp, stream)
             : moe_permute_fwd(x, x_dtype, pos_to_row, R, H, k, xp, stream);
  if (rc) return rc;
  rc = moe_gemm_gateup_swiglu_fwd(xp, w1, w3, offs, E, R, H, I, nullptr, nullptr, act, stream);
  if (rc) return rc;
  rc = moe_gemm_down_fwd(act, w2, offs, E, R, H, I, y, stream);
  if (rc) return rc;
  return moe_combine_fwd(y, gates, row_to_pos, T, H, k, out, out_dtype, stream);
}
