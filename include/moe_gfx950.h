/*
 * moe_gfx950.h -- C ABI of libmoe_gfx950.so: the MoE expert path for AMD MI355X (gfx950).
 *
 * The reference this replaces has no native or FFI interface of its own: its hot path is
 * the Python method `MoE.forward` (model/modules/mlp.py:95-169) plus the autograd backward
 * of the torch ops it calls.  Each entry point below replaces the group of torch ops cited
 * next to it.  Citations are file:line in liangyuwang/train-large-model-from-scratch.
 *
 * Conventions
 *   - T tokens, H hidden, E (local) experts, k experts per token, R = T*k routed rows,
 *     I = expert FFN width.  Flat routed row r = t*k + j, as in mlp.py:102-104.
 *   - "pos" is a position in the expert-contiguous row order (stable sort of r by expert).
 *   - All pointers are DEVICE pointers to caller-owned, contiguous, row-major buffers that
 *     stay valid until the work enqueued on `stream` has run.  bf16 is passed as
 *     `uint16_t` storage.  `dtype` arguments: MOE_DT_BF16 or MOE_DT_F32.
 *   - Every call only enqueues kernels on `stream` (a hipStream_t passed as void*); it
 *     never synchronises, allocates, prints or throws, so it may be called from any host
 *     thread.  What the library keeps between calls is a few facts per GPU that it asks the
 *     runtime for once (the compute-unit count, "this kernel's shared-memory attribute is
 *     set", the address of the fixed scratch array of moe_histogram_scan_static), looked up
 *     by the device that is current at the call; no result depends on an earlier call.
 *   - Return value: 0 on success; a positive hipError_t if a launch failed; a negative
 *     MOE_ERR_* code if an argument check failed (nothing is enqueued then).
 *   - Alignment: H and I must be multiples of 8 (rows are moved as 16-byte vectors) and
 *     every pointer 16-byte aligned.
 *   - Limits: E <= MOE_MAX_EXPERTS for routing and dispatch, E <= 1024 for the GEMMs,
 *     k <= MOE_MAX_TOPK, R <= 2^30, H and I <= 65536, and fewer than 2^31 output tiles per
 *     GEMM ((R/256 + E + 1) * ceil(max(H, I)/128)).  Buffers may exceed 4 GiB.
 */
#ifndef MOE_GFX950_H
#define MOE_GFX950_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MOE_DT_BF16 0
#define MOE_DT_F32 1

#define MOE_ERR_NULL (-1)      /* a required pointer is NULL */
#define MOE_ERR_SHAPE (-2)     /* a size is negative, zero where not allowed, or misaligned */
#define MOE_ERR_LIMIT (-3)     /* a size exceeds what the kernels support (E, k limits) */
#define MOE_ERR_DTYPE (-4)     /* unknown dtype code */
#define MOE_ERR_WORKSPACE (-5) /* workspace too small */
#define MOE_ERR_ALIGN (-6)     /* pointer not 16-byte aligned */

#define MOE_MAX_EXPERTS 512 /* router / dispatch kernels hold E/64 values per lane */
#define MOE_MAX_TOPK 64

/* Library / ABI version (major*100 + minor). */
int moe_abi_version(void);

/* ---- routing ------------------------------------------------------------------------
 * Replaces `torch.topk(gate_logits, k)` + `F.softmax(weights)` (mlp.py:101-103).
 * logits [T,E] (bf16 or f32); optional bias f32 [E] added to the logits in fp32 (NULL for the
 * reference behaviour): selection AND the softmax over the selected values use logit + bias.
 * Ties: the lower expert index wins; slots are in
 * descending-logit order.  ids_out int32 [T*k], gates_out f32 [T*k]. */
int moe_router_topk_fwd(const void* logits, int logits_dtype, const float* bias, int64_t T,
                        int64_t E, int64_t k, int32_t* ids_out, float* gates_out,
                        void* stream);

/* Backward of the softmax-over-k and of the top-k gather (autograd of mlp.py:101-102):
 * dlogits [T,E] (dtype) = scatter(gates * (dgates - sum_j gates*dgates)), zero elsewhere. */
int moe_router_topk_bwd(const float* gates, const float* dgates, const int32_t* ids,
                        int64_t T, int64_t E, int64_t k, void* dlogits, int dlogits_dtype,
                        void* stream);

/* ---- dispatch -----------------------------------------------------------------------
 * Replaces `bincount` + `cumsum` + the two `argsort`s and their inverses
 * (mlp.py:106-110, 122-127, 160, 163) with one stable counting sort.
 * ids int32 [R] in [0,E).  counts int32 [E]; offs int32 [E+1] (offs[0]=0, offs[e+1] is the
 * reference's inclusive `offs[e]`); pos_to_row int32 [R]; row_to_pos int32 [R].
 * workspace: moe_dispatch_workspace_bytes(R, E) bytes of device scratch. */
int64_t moe_dispatch_workspace_bytes(int64_t R, int64_t E);
int moe_histogram_scan(const int32_t* ids, int64_t R, int64_t E, int32_t* counts,
                       int32_t* offs, int32_t* pos_to_row, int32_t* row_to_pos,
                       void* workspace, int64_t workspace_bytes, void* stream);
/* The same, and *bad_ids (device int32, may be NULL) receives the number of ids outside [0,E).
 * Such a row is counted and placed with the nearest valid expert (0 or E-1), so that the
 * permutation stays a bijection and no kernel downstream reads out of bounds; a caller that
 * takes ids from outside (mlp.py:122, `received_experts` after the all-to-all) reads the count
 * when it next synchronises anyway and rejects the step if it is not zero.  (The reference's
 * bincount/argsort would raise or misplace silently on such ids.) */
int moe_histogram_scan_checked(const int32_t* ids, int64_t R, int64_t E, int32_t* counts,
                               int32_t* offs, int32_t* pos_to_row, int32_t* row_to_pos,
                               int32_t* bad_ids, void* workspace, int64_t workspace_bytes,
                               void* stream);

/* moe_histogram_scan_checked without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory at the
 * point of the call (code under HIP graph capture, serving loops with a frozen memory plan,
 * harnesses that forbid hipMalloc).  The per-wave histograms go to a fixed array of
 * moe_static_scratch_bytes() (4 MiB) that the library holds in every GPU's memory until the
 * process ends; MOE_ERR_WORKSPACE if moe_dispatch_workspace_bytes(R, E) exceeds it, i.e. if
 * R > moe_static_scratch_max_rows(E) = floor(4 MiB / (4 * (E+1))) * 256: 523 264 routed rows at
 * 512 experts, 4 129 536 at 64, 29 826 048 at 8.
 * RACE: all calls on one GPU share that one array.  Two such calls that overlap in time on one GPU
 * (different streams, host threads whose streams are not ordered, graphs replayed concurrently)
 * overwrite each other's histograms and return wrong permutations WITHOUT an error code; calls
 * ordered on one stream do not.  moe_static_scratch_bytes() is also the set-up call: it looks the
 * array's address up on the current device, so a caller that asks for the size before it starts
 * capturing a graph leaves no runtime query for the first moe_histogram_scan_static.  Results are
 * bit-identical to moe_histogram_scan_checked. */
int64_t moe_static_scratch_bytes(void);
int64_t moe_static_scratch_max_rows(int64_t E);
int moe_histogram_scan_static(const int32_t* ids, int64_t R, int64_t E, int32_t* counts,
                              int32_t* offs, int32_t* pos_to_row, int32_t* row_to_pos,
                              int32_t* bad_ids, void* stream);

/* Replaces `repeat_interleave(k)` + the two row gathers (mlp.py:104, 108, 124):
 * xp[pos,:] = bf16(x[pos_to_row[pos] / k, :]).  x [T,H] (x_dtype), xp bf16 [R,H]. */
int moe_permute_fwd(const void* x, int x_dtype, const int32_t* pos_to_row, int64_t R,
                    int64_t H, int64_t k, uint16_t* xp, void* stream);
/* The same result from the inverse map, token by token: x[t,:] is read once and written to
 * xp[row_to_pos[t*k+j],:] for j < k (faster when k > 1: one read feeds k stores).  Every
 * position of xp must be some routed row's place, i.e. row_to_pos is a permutation of T*k. */
int moe_permute_fwd_scatter(const void* x, int x_dtype, const int32_t* row_to_pos, int64_t T,
                            int64_t H, int64_t k, uint16_t* xp, void* stream);

/* Backward of the above (index-gather and repeat_interleave backward):
 * dx[t,:] = sum_{j<k} dxp[row_to_pos[t*k+j], :] (+ addend[t,:] if addend != NULL), summed
 * in fp32 in slot order.  dxp bf16 [R,H]; addend/dx [T,H] of dx_dtype. */
int moe_permute_bwd(const uint16_t* dxp, const int32_t* row_to_pos, const void* addend,
                    int64_t T, int64_t H, int64_t k, void* dx, int dx_dtype, void* stream);

/* The same with an addend of its own dtype (bf16 addend into an fp32 dx, or equal dtypes): the
 * router path's input gradient dlogits*Wr, a bf16 library product, joins the k-row sum in one
 * pass instead of in a separate addition. */
int moe_permute_bwd_addend(const uint16_t* dxp, const int32_t* row_to_pos, const void* addend,
                           int addend_dtype, int64_t T, int64_t H, int64_t k, void* dx,
                           int dx_dtype, void* stream);

/* ---- expert FFN ---------------------------------------------------------------------
 * Replace the three zero-padded `torch.bmm`s + SiLU + product (mlp.py:144-158) with
 * grouped GEMMs over the ragged per-expert row ranges offs[e]..offs[e+1] (empty experts
 * allowed).  bf16 operands, fp32 accumulation, bf16 results.
 * gate/up:  g = xp*W1^T, u = xp*W3^T, act = silu(g)*u.  xp [R,H]; w1,w3 [E,I,H];
 *           g,u (optional, NULL to skip; both or neither) and act: [R,I]. */
int moe_gemm_gateup_swiglu_fwd(const uint16_t* xp, const uint16_t* w1, const uint16_t* w3,
                               const int32_t* offs, int64_t E, int64_t R, int64_t H,
                               int64_t I, uint16_t* g, uint16_t* u, uint16_t* act,
                               void* stream);
/* down:     y = act*W2^T.  act [R,I]; w2 [E,H,I]; y [R,H]. */
int moe_gemm_down_fwd(const uint16_t* act, const uint16_t* w2, const int32_t* offs, int64_t E,
                      int64_t R, int64_t H, int64_t I, uint16_t* y, void* stream);

/* Backward of the down projection w.r.t. its input, fused with the SwiGLU backward
 * (autograd of mlp.py:156-157): dact = dy*W2; dg = dact*u*silu'(g); du = dact*silu(g).
 * dyp [R,H]; w2 [E,H,I]; g,u [R,I] saved by the forward; dg,du [R,I]. */
int moe_gemm_dgrad_down_swiglu_bwd(const uint16_t* dyp, const uint16_t* w2, const uint16_t* g,
                                   const uint16_t* u, const int32_t* offs, int64_t E,
                                   int64_t R, int64_t H, int64_t I, uint16_t* dg,
                                   uint16_t* du, void* stream);
/* The same, and on the way the gate gradients' raw material: dgate_part[b, pos] = sum over the
 * 64-column block b of dact[pos,:]*act[pos,:] (act = silu(g)*u in fp32).  With dyp = gate*dy the
 * blocks of a row add up to gate * <dy[token], y[pos]>, so the backward pass need not read y
 * (mlp.py:166 backward).  dgate_part fp32 [moe_dgate_blocks(I), R], every entry written. */
int64_t moe_dgate_blocks(int64_t I);
int moe_gemm_dgrad_down_swiglu_bwd_dgate(const uint16_t* dyp, const uint16_t* w2, const uint16_t* g,
                                         const uint16_t* u, const int32_t* offs, int64_t E,
                                         int64_t R, int64_t H, int64_t I, uint16_t* dg,
                                         uint16_t* du, float* dgate_part, void* stream);
/* dgates[r] = (sum_b dgate_part[b, row_to_pos[r]]) / gates[r]  (0 where the gate is 0), r in
 * routed order t*k+j; blocks added in ascending order (reproducible). */
int moe_dgates_from_blocks(const float* dgate_part, int64_t blocks, const float* gates,
                           const int32_t* row_to_pos, int64_t R, float* dgates, void* stream);
/* The same result from the inverse map (pos_to_row): positions are walked in order, so the
 * blocks are read coalesced and only the 4-byte results are scattered (mlp.py:166 backward). */
int moe_dgates_from_blocks_by_pos(const float* dgate_part, int64_t blocks, const float* gates,
                                  const int32_t* pos_to_row, int64_t R, float* dgates, void* stream);
/* g and u in a layout private to the library.  Nothing but the SwiGLU backward reads the two
 * pre-activation planes the forward saves (mlp.py:154-156 under autograd keeps them as [R, I]
 * tensors), so they need not be rows: gu_blocked holds one 4 KB record per 32 x 32 block of every
 * 256-row tile of the expert-contiguous rows, g and u of the block together, each in the order in
 * which a wavefront's matrix-core accumulators hold it.  The forward kernel stores the records
 * straight from its registers and the backward kernel loads them straight into the layout it
 * computes in; act, dg, du and dgate_part are the same bits as from the row-major entry points.
 * The buffer is opaque to the caller: moe_gu_blocked_bytes(R, E, I) bytes (it depends on R, E and
 * I only, never on the routing: (ceil(R/256) + E) * 256 rows are provided for), 16-byte aligned,
 * written by moe_gemm_gateup_swiglu_fwd_blocked and valid for moe_gemm_dgrad_down_swiglu_bwd_blocked
 * with the same offs, E, R and I.  dg and du [R, ld_out] rows (ld_out = 0 means I; 2*I with
 * du = dg + I gives the side-by-side buffer of moe_gemm_wgrad_pair); dgate_part may be NULL. */
int64_t moe_gu_blocked_bytes(int64_t R, int64_t E, int64_t I);
int moe_gemm_gateup_swiglu_fwd_blocked(const uint16_t* xp, const uint16_t* w1, const uint16_t* w3,
                                       const int32_t* offs, int64_t E, int64_t R, int64_t H,
                                       int64_t I, void* gu_blocked, uint16_t* act, void* stream);
int moe_gemm_dgrad_down_swiglu_bwd_blocked(const uint16_t* dyp, const uint16_t* w2,
                                           const void* gu_blocked, const int32_t* offs, int64_t E,
                                           int64_t R, int64_t H, int64_t I, uint16_t* dg,
                                           uint16_t* du, int64_t ld_out, float* dgate_part,
                                           void* stream);
/* Test hook (no counterpart in the reference).  The four row-ragged products (gate/up, down and
 * their two input gradients) run on 256-row tiles, or on 128-row tiles when the launch has too few
 * large tiles for half of the compute units; the choice is made from R, E and the
 * output width alone.  moe_gemm_force_row_tile(128 or 256) forces one of them for every later
 * call, 0 restores the automatic choice; the previous setting is returned.  Process-wide and not
 * synchronised with calls in flight on other host threads.  No result depends on the choice:
 * every output element is accumulated over k in the same order on both tile heights, so all
 * outputs (the gate gradients' block sums included) are the same bits either way. */
int moe_gemm_force_row_tile(int rows);
/* Backward of gate/up w.r.t. the rows (autograd of mlp.py:154-155): dxp = dg*W1 + du*W3. */
int moe_gemm_dgrad_gateup(const uint16_t* dg, const uint16_t* du, const uint16_t* w1,
                          const uint16_t* w3, const int32_t* offs, int64_t E, int64_t R,
                          int64_t H, int64_t I, uint16_t* dxp, void* stream);
/* Weight gradients (autograd of mlp.py:154-157 w.r.t. the weights), one call per stack:
 * dw[e] (+)= a[rows of e, :]^T * b[rows of e, :],  a [R,M], b [R,N], dw [E,M,N] of
 * dw_dtype.  Experts without rows get exact zeros (or are left untouched when
 * accumulate != 0).  The reduction order over rows is fixed: results are reproducible. */
int moe_gemm_wgrad(const uint16_t* a, const uint16_t* b, const int32_t* offs, int64_t E,
                   int64_t R, int64_t M, int64_t N, void* dw, int dw_dtype, int accumulate,
                   void* stream);

/* The gate and up halves of the backward in one buffer.  dgu bf16 [R, 2I] holds each row's dg and
 * du side by side ([dg row | du row]); then dgu^T * xp is ONE grouped weight-gradient product
 * whose result rows 0..I-1 are dW1 and I..2I-1 are dW3: one launch instead of two, xp read once
 * per column tile (autograd of mlp.py:154-155 w.r.t. both weights).  The three calls compute what
 * moe_gemm_dgrad_down_swiglu_bwd[_dgate] (dgate_part may be NULL), moe_gemm_dgrad_gateup and two
 * moe_gemm_wgrad calls compute, bit for bit.  moe_gemm_wgrad_pair needs I % 256 == 0
 * (MOE_ERR_SHAPE otherwise: take the separate calls on dgu's two column halves). */
int moe_gemm_dgrad_down_swiglu_bwd_packed(const uint16_t* dyp, const uint16_t* w2, const uint16_t* g,
                                          const uint16_t* u, const int32_t* offs, int64_t E, int64_t R,
                                          int64_t H, int64_t I, uint16_t* dgu, float* dgate_part,
                                          void* stream);
int moe_gemm_dgrad_gateup_packed(const uint16_t* dgu, const uint16_t* w1, const uint16_t* w3,
                                 const int32_t* offs, int64_t E, int64_t R, int64_t H, int64_t I,
                                 uint16_t* dxp, void* stream);
int moe_gemm_wgrad_pair(const uint16_t* dgu, const uint16_t* xp, const int32_t* offs, int64_t E,
                        int64_t R, int64_t I, int64_t H, void* dw1, void* dw3, int dw_dtype,
                        int accumulate, void* stream);

/* Row segments for a weight gradient whose output has too few tiles to fill the chip: every
 * expert's row range is cut into S equal parts, seg[e*S+s] = offs[e] + (offs[e+1]-offs[e])*s/S,
 * seg[E*S] = offs[E].  moe_gemm_wgrad over seg with E*S "experts" and fp32 output gives S
 * partial sums per expert, to be added in a fixed order.  E*S <= 1024.  (No counterpart in
 * the reference, whose bmm does not split the contraction.) */
int moe_segment_offsets(const int32_t* offs, int64_t E, int64_t S, int32_t* seg, void* stream);
/* The same idea with segments of bounded length, for skewed routing: expert e is cut into
 * ceil(n_e / L) equal parts, so that an expert with 40 % of the rows gets 40 % of the segments and
 * the longest contraction of the launch is L rows whatever the routing.  Segments are numbered
 * expert by expert: seg_start int32 [E+1] (seg_start[e] = e's first segment, seg_start[E] = how many
 * are used), seg int32 [S_max+1] with S_max = moe_segments_by_length_max(R, E, L) = ceil(R/L) + E
 * (a bound that holds for every routing; the slots past the used ones are empty segments at the end
 * of the rows).  moe_gemm_wgrad over seg with S_max "experts" and fp32 output gives the partial
 * sums; moe_wgrad_reduce_segments adds each expert's partials in ascending order (reproducible)
 * into dw [E,M,N] of dw_dtype: dw[e] (+)= sum_s part[s], exact zeros for experts without rows
 * (left untouched when accumulate != 0).  S_max <= 1024.  (No counterpart in the reference.) */
int64_t moe_segments_by_length_max(int64_t R, int64_t E, int64_t L);
int moe_segment_offsets_by_length(const int32_t* offs, int64_t E, int64_t L, int64_t S_max,
                                  int32_t* seg, int32_t* seg_start, void* stream);
int moe_wgrad_reduce_segments(const float* part, const int32_t* seg_start, int64_t E, int64_t M,
                              int64_t N, void* dw, int dw_dtype, int accumulate, void* stream);

/* ---- combine ------------------------------------------------------------------------
 * Replaces the un-sorts, the gate scaling and the sum over k (mlp.py:160-167):
 * out[t,:] = sum_{j<k} gates[t*k+j] * y[row_to_pos[t*k+j], :], fp32, slot order j=0..k-1.
 * gates may be NULL (all ones; with k=1 this is a pure un-permute).  out [T,H] (dtype). */
int moe_combine_fwd(const uint16_t* y, const float* gates, const int32_t* row_to_pos,
                    int64_t T, int64_t H, int64_t k, void* out, int out_dtype, void* stream);
/* The same with the caller's residual add folded in (model/gpt.py:33, `x = x + mlp_out[0]`):
 * out[t,:] = residual[t,:] + sum_j ...; residual [T,H] of out_dtype, may alias out. */
int moe_combine_fwd_residual(const uint16_t* y, const float* gates, const int32_t* row_to_pos,
                             const void* residual, int64_t T, int64_t H, int64_t k, void* out,
                             int out_dtype, void* stream);
/* Backward: dyp[pos,:] = bf16(gates[r] * dy[r/k,:]) with r = pos_to_row[pos];
 * dgates[r] = <dy[r/k,:], y[pos,:]>.  y and dgates are given together or both NULL (then only
 * dyp is made: the gate gradients can be had from moe_gemm_dgrad_down_swiglu_bwd_dgate instead);
 * gates may be NULL as well (all ones: a pure permutation of dy rows).  dy [T,H] (dtype). */
int moe_combine_bwd(const void* dy, int dy_dtype, const uint16_t* y, const float* gates,
                    const int32_t* pos_to_row, int64_t R, int64_t H, int64_t k,
                    uint16_t* dyp, float* dgates, void* stream);

/* The same result (bit for bit) from the inverse map, token by token: dy[t,:] is read once for
 * the token's k routed rows.  H <= 2048 (the row is held in registers); wider rows take
 * moe_combine_bwd. */
int moe_combine_bwd_by_token(const void* dy, int dy_dtype, const uint16_t* y, const float* gates,
                             const int32_t* row_to_pos, int64_t T, int64_t H, int64_t k,
                             uint16_t* dyp, float* dgates, void* stream);

/* ---- the step before the layer ---------------------------------------------------------
 * The caller's pre-norm (model/gpt.py:32, `self.mlp(self.ln_2(x))`; the reference's
 * `LayerNorm.forward`, model/modules/norm.py:14-19, an RMSNorm in fp32 with a weight) fused with
 * the bf16 rounding every consumer inside the layer applies (autocast at mlp.py:100, :154-155):
 *   xn[t,:] = bf16(weight * to_x_dtype(x[t,:] * rstd[t])),  rstd[t] = rsqrt(mean(x[t,:]^2) + eps).
 * x [T,H] (bf16 or fp32), weight fp32 [H], xn bf16 [T,H], rstd fp32 [T].  H % 8 == 0, H <= 8192. */
int moe_rmsnorm_fwd(const void* x, int x_dtype, const float* weight, float eps, int64_t T,
                    int64_t H, uint16_t* xn, float* rstd, void* stream);
/* The same normalisation with the router behind it in one kernel (model/gpt.py:32 feeding
 * mlp.py:100-103): besides xn and rstd it leaves the router logits bf16(xn * router_weight^T)
 * [T,E] (what the layer returns under the reference's bf16 autocast), and the top-k ids and gates
 * selected on them exactly as moe_router_topk_fwd would (no bias).  The normalised rows are not read a
 * second time for the router product.  router_weight bf16 [E,H].  Supported shapes:
 * moe_rmsnorm_router_supported(H, E, k) != 0 (H % 32 == 0, H <= 4096, E % 16 == 0, E <= 128);
 * otherwise MOE_ERR_LIMIT and the caller runs the three separate steps.  The logits come from a
 * different summation order than a library product's, so single bf16 logits may differ from it
 * by one unit in the last place; ids and gates are consistent with the logits returned here. */
int moe_rmsnorm_router_supported(int64_t H, int64_t E, int64_t k);
int moe_rmsnorm_router_fwd(const void* x, int x_dtype, const float* weight, float eps,
                           const uint16_t* router_weight, int64_t T, int64_t H, int64_t E, int64_t k,
                           uint16_t* xn, float* rstd, uint16_t* logits, int32_t* ids, float* gates,
                           void* stream);
/* Backward of the above (autograd of norm.py:14-19), with the two gradient contributions of
 * xn summed on the way in and the residual branch's gradient added on the way out:
 *   g = d1 + d2;  xhat = x*rstd;  dx = dres + rstd * (weight*g - xhat * mean(weight*g*xhat));
 *   dweight = sum_t g[t,:]*xhat[t,:]   (fixed summation order: reproducible).
 * d1 [T,H] (bf16 or fp32); d2 bf16 [T,H] or NULL; dres [T,H] of x_dtype or NULL; dx [T,H] of
 * x_dtype (may alias dres); dweight fp32 [H]; workspace of moe_rmsnorm_bwd_workspace_bytes. */
int64_t moe_rmsnorm_bwd_workspace_bytes(int64_t T, int64_t H);
int moe_rmsnorm_bwd(const void* x, int x_dtype, const float* weight, const float* rstd,
                    const void* d1, int d1_dtype, const uint16_t* d2, const void* dres, int64_t T,
                    int64_t H, void* dx, float* dweight, void* workspace, int64_t workspace_bytes,
                    void* stream);

/* ---- weight precision ---------------------------------------------------------------
 * fp32 master weights -> bf16 operands (the casts autocast inserts before each bmm,
 * mlp.py:154-157 under trainer.py:209-211). */
int moe_cast_f32_bf16(const float* src, uint16_t* dst, int64_t n, void* stream);

/* ---- the forward pass in one call ---------------------------------------------------
 * mlp.py:101-167 for a caller that wants only the output (inference, evaluation, a forward
 * under no_grad): routing, dispatch, row gather, both grouped GEMMs and the combine enqueued
 * back to back, every intermediate in `workspace` (moe_ffn_forward_workspace_bytes, 256-byte
 * aligned pieces; contents unspecified afterwards).  x [T,H] and logits [T,E] bf16 or f32, bias
 * f32 [E] or NULL, weights bf16 as stored, out [T,H] of out_dtype.  The same kernels in the same
 * order as the separate entry points: the same bits. */
int64_t moe_ffn_forward_workspace_bytes(int64_t T, int64_t H, int64_t E, int64_t I, int64_t k);
int moe_ffn_forward(const void* x, int x_dtype, const void* logits, int logits_dtype,
                    const float* bias, const uint16_t* w1, const uint16_t* w3, const uint16_t* w2,
                    int64_t T, int64_t H, int64_t E, int64_t I, int64_t k, void* out, int out_dtype,
                    void* workspace, int64_t workspace_bytes, void* stream);

/* ---- the path in fp32 ---------------------------------------------------------------
 * For a layer that runs without autocast on fp32 tensors: the reference then keeps every
 * step of mlp.py:104-169 in fp32 (the three bmm's of :154-157 included) and so do these
 * entry points.  Routing and dispatch are the entries above (fp32 logits).  Expert-contiguous
 * buffers are fp32 here: xp, dyp, dxp, y [R,H]; g, u, act, dact, dg, du [R,I].  H and I must be
 * multiples of 4 (16-byte accesses); weights are the fp32 parameters themselves.  Limits as
 * above (R <= 2^30, widths <= 65536, E <= 1024 for the GEMMs) and fewer than 2^31 output tiles
 * of 64 x 64 per GEMM. */

/* mlp.py:104-131 (repeat_interleave + both sorts): xp[pos,:] = x[pos_to_row[pos] / k, :]. */
int moe_f32_gather_rows(const float* x, const int32_t* pos_to_row, int64_t T, int64_t R, int64_t H,
                        int64_t k, float* xp, void* stream);
/* mlp.py:160-169: out[t,:] = sum_j gates[t*k+j] * y[row_to_pos[t*k+j],:], j ascending.
 * gates may be NULL (all ones; with k = 1 a pure un-permute), here and in the backward. */
int moe_f32_combine_fwd(const float* y, const float* gates, const int32_t* row_to_pos, int64_t T,
                        int64_t H, int64_t k, float* out, void* stream);
/* Its backward: dyp[pos,:] = gates[row] * dy[row / k,:] and, unless dgates is NULL,
 * dgates[row] = <dy[row / k,:], y[pos,:]> (row = pos_to_row[pos]; y may be NULL with dgates). */
int moe_f32_combine_bwd(const float* dy, const float* y, const float* gates, const int32_t* pos_to_row,
                        int64_t T, int64_t R, int64_t H, int64_t k, float* dyp, float* dgates,
                        void* stream);
/* Backward of the gather: dx[t,:] = sum_j dxp[row_to_pos[t*k+j],:], j ascending. */
int moe_f32_permute_bwd(const float* dxp, const int32_t* row_to_pos, int64_t T, int64_t H, int64_t k,
                        float* dx, void* stream);
/* mlp.py:156: act = silu(g) * u over n elements (n a multiple of 4), and its backward
 * dg = dact * u * silu'(g), du = dact * silu(g). */
int moe_f32_swiglu_fwd(const float* g, const float* u, int64_t n, float* act, void* stream);
int moe_f32_swiglu_bwd(const float* dact, const float* g, const float* u, int64_t n, float* dg,
                       float* du, void* stream);
/* The bmm's of mlp.py:154-157 and their input gradients over ragged expert rows (no padding):
 * c[r,:] (+)= a[r,:] x B_e for the rows r of expert e; a [R,K], c [R,N], b [E,N,K] when
 * b_k_contiguous (c = a b_e^T: x W1^T, x W3^T, act W2^T) or [E,K,N] otherwise (c = a b_e:
 * dy W2, dg W1, du W3).  accumulate != 0 adds into c. */
int moe_f32_gemm_rows(const float* a, const float* b, const int32_t* offs, int64_t E, int64_t R,
                      int64_t N, int64_t K, int b_k_contiguous, float* c, int accumulate, void* stream);
/* Their weight gradients: dw[e] (+)= a[rows of e]^T b[rows of e]; a [R,M], b [R,N], dw [E,M,N].
 * Experts without rows get exact zeros (are left untouched when accumulating). */
int moe_f32_gemm_wgrad(const float* a, const float* b, const int32_t* offs, int64_t E, int64_t R,
                       int64_t M, int64_t N, float* dw, int accumulate, void* stream);
/* Test hook (no counterpart in the reference): the two fp32 GEMM entries choose 64 x 64 or
 * 128 x 128 output tiles from the shapes; 64 or 128 forces one, 0 restores the choice.  Returns
 * the previous setting.  Process-wide, not synchronised. */
int moe_f32_gemm_force_tile(int t);

#ifdef __cplusplus
}
#endif
#endif /* MOE_GFX950_H */
