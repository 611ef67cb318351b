"""Python wrappers over the C ABI: allocate outputs with torch, pass raw device pointers
and the current HIP stream, check the return code.  One function per exported kernel group.

Every function requires CUDA(HIP) tensors; nothing here computes on the host.
"""
from __future__ import annotations

import torch

from . import lib as _lib
from .lib import DT_BF16, DT_F32


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return DT_BF16
    if t.dtype == torch.float32:
        return DT_F32
    raise TypeError(f"unsupported dtype {t.dtype}: the MoE kernels take bf16 or fp32")


def _p(t: torch.Tensor | None):
    if t is None:
        return None
    if not t.is_cuda:
        raise RuntimeError("the MoE kernels need GPU tensors (no CPU path exists)")
    if not t.is_contiguous():
        raise RuntimeError("the MoE kernels need contiguous tensors")
    return t.data_ptr()


def dense(t: torch.Tensor) -> torch.Tensor:
    """Contiguous and 16-byte aligned, as the kernels need their buffers: a copy only for a
    strided view or a view that starts in the middle of an aligned block."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """Handle of torch's current stream.  Through torch's raw accessor where it exists: building
    the Python stream object costs about 10 us per launch, which is the whole budget of a
    launch in the small configurations."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def launch_observer():
    """The object installed as the library's launch observer (a profiling aid), or None."""
    return _lib.load().observer


def router_topk(logits: torch.Tensor, k: int, bias: torch.Tensor | None = None):
    """logits [T,E] (bf16/fp32) -> ids int32 [T*k], gates fp32 [T*k]."""
    T, E = logits.shape
    ids = torch.empty(T * k, dtype=torch.int32, device=logits.device)
    gates = torch.empty(T * k, dtype=torch.float32, device=logits.device)
    _lib.load().call("moe_router_topk_fwd", _p(logits), _dt(logits), _p(bias), T, E, k,
                     _p(ids), _p(gates), _stream())
    return ids, gates


def router_topk_bwd(gates, dgates, ids, T: int, E: int, k: int, dtype: torch.dtype):
    dlogits = torch.empty(T, E, dtype=dtype, device=gates.device)
    _lib.load().call("moe_router_topk_bwd", _p(gates), _p(dgates), _p(ids), T, E, k,
                     _p(dlogits), _dt(dlogits), _stream())
    return dlogits


def histogram_scan(ids: torch.Tensor, E: int, return_bad: bool = False):
    """ids int32 [R] -> counts int32 [E], offs int32 [E+1], pos_to_row, row_to_pos int32 [R].
    With `return_bad` a fifth tensor (int32 [1], on the device) holds the number of ids outside
    [0, E); reading it is the caller's business (it costs a synchronisation)."""
    R = ids.numel()
    dev = ids.device
    L = _lib.load()
    ws_bytes = L.cdll.moe_dispatch_workspace_bytes(R, E)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    offs = torch.empty(E + 1, dtype=torch.int32, device=dev)
    pos_to_row = torch.empty(R, dtype=torch.int32, device=dev)
    row_to_pos = torch.empty(R, dtype=torch.int32, device=dev)
    bad = torch.empty(1, dtype=torch.int32, device=dev) if return_bad else None
    L.call("moe_histogram_scan_checked", _p(ids), R, E, _p(counts), _p(offs), _p(pos_to_row),
           _p(row_to_pos), _p(bad), _p(ws), ws.numel(), _stream())
    if return_bad:
        return counts, offs, pos_to_row, row_to_pos, bad
    return counts, offs, pos_to_row, row_to_pos


def permute_fwd(x: torch.Tensor, pos_to_row: torch.Tensor, k: int,
                row_to_pos: torch.Tensor | None = None) -> torch.Tensor:
    """xp[pos] = bf16(x[pos_to_row[pos] // k]).  With the inverse map also given (and k > 1) the
    rows are written token by token instead of gathered: same result, one read per token."""
    R, H = pos_to_row.numel(), x.shape[-1]
    xp = torch.empty(R, H, dtype=torch.bfloat16, device=x.device)
    if row_to_pos is not None and k > 1:
        _lib.load().call("moe_permute_fwd_scatter", _p(x), _dt(x), _p(row_to_pos), R // k, H, k, _p(xp),
                         _stream())
    else:
        _lib.load().call("moe_permute_fwd", _p(x), _dt(x), _p(pos_to_row), R, H, k, _p(xp), _stream())
    return xp


def permute_bwd(dxp: torch.Tensor, row_to_pos: torch.Tensor, T: int, k: int, dtype: torch.dtype,
                addend: torch.Tensor | None = None) -> torch.Tensor:
    H = dxp.shape[-1]
    dx = torch.empty(T, H, dtype=dtype, device=dxp.device)
    if addend is not None and addend.dtype != dtype:
        if not (addend.dtype == torch.bfloat16 and dtype == torch.float32):
            raise TypeError("addend must have the output dtype, or be bf16 for an fp32 output")
        _lib.load().call("moe_permute_bwd_addend", _p(dxp), _p(row_to_pos), _p(addend), _dt(addend), T, H, k,
                         _p(dx), _dt(dx), _stream())
        return dx
    _lib.load().call("moe_permute_bwd", _p(dxp), _p(row_to_pos), _p(addend), T, H, k, _p(dx),
                     _dt(dx), _stream())
    return dx


def gemm_gateup(xp, w1, w3, offs, save_gu: bool):
    R, H = xp.shape
    E, I, _ = w1.shape
    act = torch.empty(R, I, dtype=torch.bfloat16, device=xp.device)
    g = torch.empty_like(act) if save_gu else None
    u = torch.empty_like(act) if save_gu else None
    _lib.load().call("moe_gemm_gateup_swiglu_fwd", _p(xp), _p(w1), _p(w3), _p(offs), E, R, H, I,
                     _p(g), _p(u), _p(act), _stream())
    return g, u, act


def gemm_gateup_blocked(xp, w1, w3, offs):
    """gemm_gateup for a forward pass whose g and u only the SwiGLU backward will read: they are
    left in the library's blocked layout (an opaque uint8 buffer; see include/moe_gfx950.h), which
    the forward kernel writes straight from its registers.  -> gu_blocked, act [R,I]."""
    R, H = xp.shape
    E, I, _ = w1.shape
    L = _lib.load()
    act = torch.empty(R, I, dtype=torch.bfloat16, device=xp.device)
    gu = torch.empty(max(L.cdll.moe_gu_blocked_bytes(R, E, I), 16), dtype=torch.uint8, device=xp.device)
    L.call("moe_gemm_gateup_swiglu_fwd_blocked", _p(xp), _p(w1), _p(w3), _p(offs), E, R, H, I, _p(gu), _p(act),
           _stream())
    return gu, act


def gemm_dgrad_down_blocked(dyp, w2, gu, offs, dgate_blocks: bool = False, packed: bool = False):
    """gemm_dgrad_down / gemm_dgrad_down_packed on blocked g/u: -> (dg, du, part) with `dg`, `du` [R,I], or
    (dgu, part) with dgu [R,2I] = [dg | du] when `packed`; `part` as in gemm_dgrad_down (None without
    `dgate_blocks`).  Same bits as the row-major entries."""
    R, H = dyp.shape
    E, _, I = w2.shape
    L = _lib.load()
    part = torch.empty(L.cdll.moe_dgate_blocks(I), R, dtype=torch.float32, device=dyp.device) if dgate_blocks else None
    if packed:
        dgu = torch.empty(R, 2 * I, dtype=torch.bfloat16, device=dyp.device)
        dg, du, ld = dgu, dgu[:, I:], 2 * I
    else:
        dg = torch.empty(R, I, dtype=torch.bfloat16, device=dyp.device)
        du = torch.empty_like(dg)
        ld = 0
    L.call("moe_gemm_dgrad_down_swiglu_bwd_blocked", _p(dyp), _p(w2), _p(gu), _p(offs), E, R, H, I,
           dg.data_ptr(), du.data_ptr(), ld, _p(part), _stream())
    if packed:
        return dgu, part
    return dg, du, part


def gemm_down(act, w2, offs):
    R, I = act.shape
    E, H, _ = w2.shape
    y = torch.empty(R, H, dtype=torch.bfloat16, device=act.device)
    _lib.load().call("moe_gemm_down_fwd", _p(act), _p(w2), _p(offs), E, R, H, I, _p(y), _stream())
    return y


def gemm_dgrad_down(dyp, w2, g, u, offs, dgate_blocks: bool = False):
    """-> dg, du [R,I] bf16; with `dgate_blocks` also the fp32 [blocks, R] partial sums of
    <dact, act> per row (see dgates_from_blocks)."""
    R, H = dyp.shape
    E, _, I = w2.shape
    dg = torch.empty(R, I, dtype=torch.bfloat16, device=dyp.device)
    du = torch.empty_like(dg)
    L = _lib.load()
    if dgate_blocks:
        part = torch.empty(L.cdll.moe_dgate_blocks(I), R, dtype=torch.float32, device=dyp.device)
        L.call("moe_gemm_dgrad_down_swiglu_bwd_dgate", _p(dyp), _p(w2), _p(g), _p(u), _p(offs),
               E, R, H, I, _p(dg), _p(du), _p(part), _stream())
        return dg, du, part
    L.call("moe_gemm_dgrad_down_swiglu_bwd", _p(dyp), _p(w2), _p(g), _p(u), _p(offs),
           E, R, H, I, _p(dg), _p(du), _stream())
    return dg, du


def dgates_from_blocks(part, gates, row_to_pos, pos_to_row=None):
    """Gate gradients dgates[r] = <dy[token of r], y[row of r]> from the per-row block sums the
    dgrad-down kernel left (they hold gate * that product).  With the inverse map also given the
    blocks are read in position order (coalesced) and the results scattered: the same values."""
    R = gates.numel()
    dgates = torch.empty(R, dtype=torch.float32, device=gates.device)
    if pos_to_row is not None:
        _lib.load().call("moe_dgates_from_blocks_by_pos", _p(part), part.shape[0], _p(gates),
                         _p(pos_to_row), R, _p(dgates), _stream())
    else:
        _lib.load().call("moe_dgates_from_blocks", _p(part), part.shape[0], _p(gates),
                         _p(row_to_pos), R, _p(dgates), _stream())
    return dgates


def gemm_dgrad_gateup(dg, du, w1, w3, offs):
    R, I = dg.shape
    E, _, H = w1.shape
    dxp = torch.empty(R, H, dtype=torch.bfloat16, device=dg.device)
    _lib.load().call("moe_gemm_dgrad_gateup", _p(dg), _p(du), _p(w1), _p(w3), _p(offs), E, R, H, I,
                     _p(dxp), _stream())
    return dxp


def gemm_wgrad(a, b, offs, E: int, dtype: torch.dtype, out: torch.Tensor | None = None):
    """dw[e] (+)= a[rows e]^T b[rows e]; a [R,M], b [R,N] -> [E,M,N].  `out` accumulates."""
    R, M = a.shape
    N = b.shape[1]
    acc = out is not None
    if out is None:
        out = torch.empty(E, M, N, dtype=dtype, device=a.device)
    _lib.load().call("moe_gemm_wgrad", _p(a), _p(b), _p(offs), E, R, M, N, _p(out), _dt(out),
                     1 if acc else 0, _stream())
    return out


def gemm_dgrad_down_packed(dyp, w2, g, u, offs, dgate_blocks: bool = False):
    """gemm_dgrad_down with dg and du side by side in one buffer: -> dgu bf16 [R, 2I] (row =
    [dg row | du row]) and, with `dgate_blocks`, the block sums (else None)."""
    R, H = dyp.shape
    E, _, I = w2.shape
    dgu = torch.empty(R, 2 * I, dtype=torch.bfloat16, device=dyp.device)
    L = _lib.load()
    part = torch.empty(L.cdll.moe_dgate_blocks(I), R, dtype=torch.float32, device=dyp.device) if dgate_blocks else None
    L.call("moe_gemm_dgrad_down_swiglu_bwd_packed", _p(dyp), _p(w2), _p(g), _p(u), _p(offs), E, R, H, I,
           _p(dgu), _p(part), _stream())
    return dgu, part


def gemm_dgrad_gateup_packed(dgu, w1, w3, offs):
    R = dgu.shape[0]
    E, I, H = w1.shape
    dxp = torch.empty(R, H, dtype=torch.bfloat16, device=dgu.device)
    _lib.load().call("moe_gemm_dgrad_gateup_packed", _p(dgu), _p(w1), _p(w3), _p(offs), E, R, H, I, _p(dxp), _stream())
    return dxp


def gemm_wgrad_pair(dgu, xp, offs, E: int, dtype: torch.dtype, out1=None, out3=None):
    """dW1[e] (+)= dg[rows e]^T xp[rows e], dW3[e] (+)= du[rows e]^T xp[rows e] from dgu = [dg | du] in
    one launch; I % 256 == 0.  `out1`/`out3` (both or neither) accumulate."""
    R, I2 = dgu.shape
    I, H = I2 // 2, xp.shape[1]
    acc = out1 is not None
    if not acc:
        out1 = torch.empty(E, I, H, dtype=dtype, device=dgu.device)
        out3 = torch.empty(E, I, H, dtype=dtype, device=dgu.device)
    _lib.load().call("moe_gemm_wgrad_pair", _p(dgu), _p(xp), _p(offs), E, R, I, H, _p(out1), _p(out3), _dt(out1),
                     1 if acc else 0, _stream())
    return out1, out3


def segment_offsets(offs: torch.Tensor, E: int, S: int) -> torch.Tensor:
    """offs int32 [E+1] -> int32 [E*S+1]: every expert's rows cut into S equal parts."""
    seg = torch.empty(E * S + 1, dtype=torch.int32, device=offs.device)
    _lib.load().call("moe_segment_offsets", _p(offs), E, S, _p(seg), _stream())
    return seg


def segment_offsets_by_length(offs: torch.Tensor, E: int, L: int, R: int):
    """offs int32 [E+1] -> (seg int32 [S_max+1], seg_start int32 [E+1], S_max): every expert's rows cut
    into ceil(n_e / L) equal parts, numbered expert by expert; S_max = ceil(R/L) + E bounds their
    number for any routing (unused slots are empty segments)."""
    L_ = _lib.load()
    S_max = int(L_.cdll.moe_segments_by_length_max(R, E, L))
    seg = torch.empty(S_max + 1, dtype=torch.int32, device=offs.device)
    seg_start = torch.empty(E + 1, dtype=torch.int32, device=offs.device)
    L_.call("moe_segment_offsets_by_length", _p(offs), E, L, S_max, _p(seg), _p(seg_start), _stream())
    return seg, seg_start, S_max


def wgrad_reduce_segments(part: torch.Tensor, seg_start: torch.Tensor, E: int, dtype: torch.dtype,
                          out: torch.Tensor | None = None):
    """part fp32 [S_max, M, N] -> dw [E, M, N]: each expert's partial sums added in ascending order;
    `out` accumulates."""
    _, M, N = part.shape
    acc = out is not None
    if out is None:
        out = torch.empty(E, M, N, dtype=dtype, device=part.device)
    _lib.load().call("moe_wgrad_reduce_segments", _p(part), _p(seg_start), E, M, N, _p(out), _dt(out),
                     1 if acc else 0, _stream())
    return out


def combine_fwd(y, gates, row_to_pos, T: int, k: int, dtype: torch.dtype):
    H = y.shape[-1]
    out = torch.empty(T, H, dtype=dtype, device=y.device)
    _lib.load().call("moe_combine_fwd", _p(y), _p(gates), _p(row_to_pos), T, H, k, _p(out),
                     _dt(out), _stream())
    return out


def combine_fwd_residual(y, gates, row_to_pos, residual: torch.Tensor, k: int):
    """residual [T,H] + the combined expert rows; same dtype as `residual`."""
    T, H = residual.shape
    out = torch.empty_like(residual)
    _lib.load().call("moe_combine_fwd_residual", _p(y), _p(gates), _p(row_to_pos), _p(residual), T, H, k,
                     _p(out), _dt(out), _stream())
    return out


def rmsnorm_fwd(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """x [T,H] (bf16/fp32), weight fp32 [H] -> xn bf16 [T,H], rstd fp32 [T]."""
    T, H = x.shape
    xn = torch.empty(T, H, dtype=torch.bfloat16, device=x.device)
    rstd = torch.empty(T, dtype=torch.float32, device=x.device)
    _lib.load().call("moe_rmsnorm_fwd", _p(x), _dt(x), _p(weight), float(eps), T, H, _p(xn), _p(rstd),
                     _stream())
    return xn, rstd


def rmsnorm_router_supported(H: int, E: int, k: int) -> bool:
    return bool(_lib.load().cdll.moe_rmsnorm_router_supported(H, E, k))


def rmsnorm_router_fwd(x: torch.Tensor, weight: torch.Tensor, eps: float, router_weight: torch.Tensor, k: int):
    """RMSNorm, router product and top-k in one kernel: x [T,H], norm weight fp32 [H], router
    weight bf16 [E,H] -> xn bf16 [T,H], rstd fp32 [T], logits bf16 [T,E], ids int32 [T*k],
    gates fp32 [T*k]."""
    T, H = x.shape
    E = router_weight.shape[0]
    dev = x.device
    xn = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    rstd = torch.empty(T, dtype=torch.float32, device=dev)
    logits = torch.empty(T, E, dtype=torch.bfloat16, device=dev)
    ids = torch.empty(T * k, dtype=torch.int32, device=dev)
    gates = torch.empty(T * k, dtype=torch.float32, device=dev)
    _lib.load().call("moe_rmsnorm_router_fwd", _p(x), _dt(x), _p(weight), float(eps), _p(router_weight), T, H, E, k,
                     _p(xn), _p(rstd), _p(logits), _p(ids), _p(gates), _stream())
    return xn, rstd, logits, ids, gates


def rmsnorm_bwd(x, weight, rstd, d1, d2=None, dres=None):
    """-> dx [T,H] (dtype of x), dweight fp32 [H]; see include/moe_gfx950.h."""
    T, H = x.shape
    L = _lib.load()
    ws = torch.empty(max(L.cdll.moe_rmsnorm_bwd_workspace_bytes(T, H), 16), dtype=torch.uint8, device=x.device)
    dx = torch.empty_like(x)
    dw = torch.empty(H, dtype=torch.float32, device=x.device)
    if dres is not None and dres.dtype != x.dtype:
        raise TypeError("dres must have the dtype of x")
    L.call("moe_rmsnorm_bwd", _p(x), _dt(x), _p(weight), _p(rstd), _p(d1), _dt(d1), _p(d2), _p(dres),
           T, H, _p(dx), _p(dw), _p(ws), ws.numel(), _stream())
    return dx, dw


def combine_bwd(dy, y, gates, pos_to_row, k: int, row_to_pos: torch.Tensor | None = None):
    """dyp[pos] = bf16(gate * dy[token of pos]), dgates[r] = <dy[token], y[pos]>.  With the
    inverse map also given, k > 1 and H <= 2048 the work is done token by token (dy read once
    per token): same bits."""
    R, H = pos_to_row.numel(), dy.shape[-1]
    dyp = torch.empty(R, H, dtype=torch.bfloat16, device=dy.device)
    dgates = torch.empty(R, dtype=torch.float32, device=dy.device) if y is not None else None
    if row_to_pos is not None and k > 1 and H <= 2048:
        _lib.load().call("moe_combine_bwd_by_token", _p(dy), _dt(dy), _p(y), _p(gates), _p(row_to_pos),
                         R // k, H, k, _p(dyp), _p(dgates), _stream())
        return dyp, dgates
    _lib.load().call("moe_combine_bwd", _p(dy), _dt(dy), _p(y), _p(gates), _p(pos_to_row), R, H, k,
                     _p(dyp), _p(dgates), _stream())
    return dyp, dgates


def cast_bf16(w: torch.Tensor) -> torch.Tensor:
    """fp32 -> bf16 copy through the library's cast kernel; bf16 input is returned as is."""
    if w.dtype == torch.bfloat16:
        return w
    out = torch.empty(w.shape, dtype=torch.bfloat16, device=w.device)
    _lib.load().call("moe_cast_f32_bf16", _p(w), _p(out), w.numel(), _stream())
    return out


def ffn_forward(x: torch.Tensor, logits: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor, w2: torch.Tensor,
                k: int, bias: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """The layer body's forward pass in one call of the library (no intermediate is kept): x [T,H]
    bf16/fp32, logits [T,E] bf16/fp32, bf16 weights -> out [T,H] of `out_dtype` (default: x's)."""
    T, H = x.shape
    E, I = w1.shape[0], w1.shape[1]
    L = _lib.load()
    out = torch.empty(T, H, dtype=out_dtype or x.dtype, device=x.device)
    nbytes = L.cdll.moe_ffn_forward_workspace_bytes(T, H, E, I, k)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=x.device)
    L.call("moe_ffn_forward", _p(x), _dt(x), _p(logits), _dt(logits), _p(bias), _p(w1), _p(w3), _p(w2),
           T, H, E, I, k, _p(out), _dt(out), _p(ws), ws.numel(), _stream())
    return out


# ---- the path in fp32 (layer called without autocast on fp32 tensors) ---------------------------

def _check_offs(offs: torch.Tensor, E: int):
    if offs.dtype != torch.int32 or offs.numel() != E + 1:
        raise ValueError(f"offs must be int32 [E + 1] = [{E + 1}], got {offs.dtype} {tuple(offs.shape)}")


def _f32(*ts):
    for t in ts:
        if t is not None and t.dtype != torch.float32:
            raise TypeError(f"the fp32 entry points take fp32 tensors, got {t.dtype}")


def f32_gather_rows(x: torch.Tensor, pos_to_row: torch.Tensor, k: int) -> torch.Tensor:
    """xp[pos] = x[pos_to_row[pos] // k], fp32 [R,H]."""
    _f32(x)
    T, H = x.shape
    R = pos_to_row.numel()
    xp = torch.empty(R, H, dtype=torch.float32, device=x.device)
    _lib.load().call("moe_f32_gather_rows", _p(x), _p(pos_to_row), T, R, H, k, _p(xp), _stream())
    return xp


def f32_combine_fwd(y: torch.Tensor, gates: torch.Tensor | None, row_to_pos: torch.Tensor, T: int, k: int):
    """out[t] = sum_j gates[t*k+j] * y[row_to_pos[t*k+j]]; gates None: all ones."""
    _f32(y, gates)
    H = y.shape[-1]
    out = torch.empty(T, H, dtype=torch.float32, device=y.device)
    _lib.load().call("moe_f32_combine_fwd", _p(y), _p(gates), _p(row_to_pos), T, H, k, _p(out), _stream())
    return out


def f32_combine_bwd(dy, y, gates, pos_to_row, k: int):
    """-> dyp fp32 [R,H], dgates fp32 [R] (None when y is None)."""
    _f32(dy, y, gates)
    T, H = dy.shape
    R = pos_to_row.numel()
    dyp = torch.empty(R, H, dtype=torch.float32, device=dy.device)
    dgates = torch.empty(R, dtype=torch.float32, device=dy.device) if y is not None else None
    _lib.load().call("moe_f32_combine_bwd", _p(dy), _p(y), _p(gates), _p(pos_to_row), T, R, H, k, _p(dyp),
                     _p(dgates), _stream())
    return dyp, dgates


def f32_permute_bwd(dxp: torch.Tensor, row_to_pos: torch.Tensor, T: int, k: int) -> torch.Tensor:
    _f32(dxp)
    H = dxp.shape[-1]
    dx = torch.empty(T, H, dtype=torch.float32, device=dxp.device)
    _lib.load().call("moe_f32_permute_bwd", _p(dxp), _p(row_to_pos), T, H, k, _p(dx), _stream())
    return dx


def f32_swiglu(g: torch.Tensor, u: torch.Tensor) -> torch.Tensor:
    _f32(g, u)
    act = torch.empty_like(g)
    _lib.load().call("moe_f32_swiglu_fwd", _p(g), _p(u), g.numel(), _p(act), _stream())
    return act


def f32_swiglu_bwd(dact, g, u):
    _f32(dact, g, u)
    dg, du = torch.empty_like(g), torch.empty_like(g)
    _lib.load().call("moe_f32_swiglu_bwd", _p(dact), _p(g), _p(u), g.numel(), _p(dg), _p(du), _stream())
    return dg, du


def f32_gemm_rows(a: torch.Tensor, b: torch.Tensor, offs: torch.Tensor, transpose_b: bool,
                  out: torch.Tensor | None = None) -> torch.Tensor:
    """Per expert e over its rows: a[rows] @ b[e].T (`transpose_b`, b [E,N,K]) or a[rows] @ b[e]
    (b [E,K,N]).  With `out` the product is added into it."""
    _f32(a, b, out)
    R, K = a.shape
    E = b.shape[0]
    N = b.shape[1] if transpose_b else b.shape[2]
    if (b.shape[2] if transpose_b else b.shape[1]) != K:
        raise ValueError(f"depth mismatch: a {tuple(a.shape)}, b {tuple(b.shape)}, transpose_b={transpose_b}")
    _check_offs(offs, E)
    if out is not None and tuple(out.shape) != (R, N):
        raise ValueError(f"out has shape {tuple(out.shape)}, the product {(R, N)}")
    c = out if out is not None else torch.empty(R, N, dtype=torch.float32, device=a.device)
    _lib.load().call("moe_f32_gemm_rows", _p(a), _p(b), _p(offs), E, R, N, K, int(transpose_b), _p(c),
                     int(out is not None), _stream())
    return c


def f32_gemm_wgrad(a: torch.Tensor, b: torch.Tensor, offs: torch.Tensor, E: int,
                   out: torch.Tensor | None = None) -> torch.Tensor:
    """dw[e] = a[rows of e].T @ b[rows of e] -> fp32 [E,M,N]; with `out` added into it."""
    _f32(a, b, out)
    R, M = a.shape
    N = b.shape[1]
    _check_offs(offs, E)
    if b.shape[0] != R or (out is not None and tuple(out.shape) != (E, M, N)):
        raise ValueError(f"shape mismatch: a {tuple(a.shape)}, b {tuple(b.shape)}, E {E}"
                         + ("" if out is None else f", out {tuple(out.shape)}"))
    dw = out if out is not None else torch.empty(E, M, N, dtype=torch.float32, device=a.device)
    _lib.load().call("moe_f32_gemm_wgrad", _p(a), _p(b), _p(offs), E, R, M, N, _p(dw), int(out is not None),
                     _stream())
    return dw
