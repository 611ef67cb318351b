"""Differentiable entry points built on the HIP kernels.

`moe_ffn`      x [T,H] + router logits [T,E] -> out [T,H]: the body of the reference's
               `MoE.forward` after the router linear (model/modules/mlp.py:101-167).
`experts_rows` rows [R,H] + local expert ids [R] -> out [R,H] in arrival order: the part
               between the two all-to-alls (mlp.py:122-161), i.e. one rank's local share.

`router_linear` x [T,H], Wr [E,H] -> logits [T,E]: the router product (mlp.py:100) with the same
               autocast rule as `nn.Linear`; its weight gradient, a 64 x 2048 x 16384 product
               in benchmark config 3 that the BLAS library has no good kernel for, runs as a
               split-k sum on the grouped weight-gradient kernel.

`prenorm_moe`  x [T,H] residual stream -> x + MoE(RMSNorm(x)) and the router logits: the caller's
               two lines around the layer (model/gpt.py:32-33) in one differentiable call.  The
               normalisation writes the bf16 rows the layer consumes in one pass over x, the
               residual add rides in the combine kernel, and in the backward pass the three
               gradient streams into x (expert path, router path, residual) meet inside the
               normalisation's backward kernel instead of in separate additions.

`moe_ffn` and `experts_rows` compute in bf16 on the matrix cores with fp32 accumulation,
whatever the input dtype; outputs and input gradients take the dtype of `x`, weight gradients
the dtype of the weights.  `moe_ffn_f32` is the same function with every step in fp32 (fp32
matrix instructions, fp32 rows): what the reference computes when it is called without autocast
on fp32 tensors.  There is no host synchronisation anywhere in either direction.

Weight gradients into `.grad` (`accumulate_into_grad=True`): the reference's trainer sums
the gradients of several micro-steps in the parameters' `.grad` (training/trainer.py:241-248),
which costs autograd one more read-add-write pass over every expert weight gradient per
micro-step.  With the option on, the weight-gradient kernel adds its result to the existing
`.grad` in its own epilogue (or creates `.grad` on the first micro-step) and autograd
receives no gradient for the three stacks.  The sums are the same numbers (one fp32 add per
element either way); what changes is that autograd hooks on these parameters no longer see
the gradient (tensor hooks are called with None, nothing reaches the accumulation node), so
a data-parallel wrapper that reduces gradients from such hooks must leave the option off.
"""
from __future__ import annotations

import torch

from . import ops
from .ops import dense as _dense


def _first_order_only():
    """Called at the top of every backward here.  The backward passes run kernels autograd cannot
    see through, so a gradient of a gradient would silently lack their terms: refuse to build a
    graph over them (grad mode is on inside a backward pass only under `create_graph=True`)."""
    if torch.is_grad_enabled():
        raise RuntimeError("the MoE kernels' backward pass is not differentiable: call backward()/grad() "
                           "without create_graph=True")


_SPLIT_ROWS = 512  # tokens per partial sum of the router weight gradient
_split_offsets = {}  # (tokens, slices, device) -> int32 slice bounds


class _RouterLinear(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda", cast_inputs=torch.bfloat16)
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return torch.nn.functional.linear(x, w)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx, dlogits):
        _first_order_only()
        x, w = ctx.saved_tensors
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = dlogits @ w
        if ctx.needs_input_grad[1]:
            dw = _router_wgrad(dlogits, x, w.dtype)
        return dx, dw


def _router_wgrad(dlogits, x, w_dtype):
    """dWr = dlogits^T x for dlogits [T,E], x [T,H]."""
    T, H = x.shape
    E = dlogits.shape[1]
    fast = (x.is_cuda and x.dtype == torch.bfloat16 and dlogits.dtype == torch.bfloat16
            and E % 8 == 0 and H % 8 == 0 and T > 0)
    if not fast:
        return (dlogits.t() @ x).to(w_dtype)
    # contraction over the tokens: slices of _SPLIT_ROWS tokens play the experts of the ragged
    # weight-gradient kernel, fp32 partials are summed in a fixed order (deterministic)
    S = min(128, (T + _SPLIT_ROWS - 1) // _SPLIT_ROWS)
    key = (T, S, x.device)
    offs = _split_offsets.get(key)
    if offs is None:  # constant for a given token count: made once
        step = (T + S - 1) // S
        offs = torch.clamp(torch.arange(S + 1, device=x.device, dtype=torch.int32) * step, max=T).to(torch.int32)
        # (not kept when made under graph capture: such a tensor lives in the graph's memory and is
        # only filled when the graph runs)
        # (entries are never dropped: a captured graph may be reading one; each is at most 129 ints)
        if not torch.cuda.is_current_stream_capturing() and len(_split_offsets) < 4096:
            _split_offsets[key] = offs
    part = ops.gemm_wgrad(_dense(dlogits), _dense(x), offs, S, torch.float32)
    return part.sum(0).to(w_dtype)


def router_linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """Router logits `x @ weight^T` (mlp.py:100) for x [..., H], weight [E, H].  Forward and
    input gradient are the library products `nn.Linear` would run, under the same autocast
    rule (bf16 operands and result inside a bf16 autocast region); the weight gradient is
    computed here (see the module docstring)."""
    lead = x.shape[:-1]
    out = _RouterLinear.apply(x.reshape(-1, x.shape[-1]), weight)
    return out.reshape(*lead, weight.shape[0])


_WGRAD_TILE = 256   # output tile edge of the weight-gradient kernel
_cu_count = {}


def _compute_units(device) -> int:
    n = _cu_count.get(device)
    if n is None:
        n = _cu_count[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return n


def _wgrad_split(E: int, M: int, N: int, device) -> int:
    """Compute units per output tile of the weight-gradient launch for [E, M, N] (at least 1).
    The kernel makes one workgroup per 256 x 256 output tile and expert; with few experts and
    small matrices that is a fraction of the chip, and under skewed routing the tiles of the
    largest expert set the time: from 2 on, the contraction is cut into row segments.  Decided
    from shapes alone (no look at the counts, no host synchronisation)."""
    tiles = E * -(-M // _WGRAD_TILE) * -(-N // _WGRAD_TILE)
    return max(1, _compute_units(device) // max(tiles, 1))


def _segment_rows(E: int, M: int, N: int, R: int, device) -> int:
    """Row segment length L for a small launch: every expert's contraction is cut into
    ceil(n_e / L) equal parts, so that the (ceil(R/L) + E) x tiles jobs about fill the compute
    units once and none contracts over more than L rows, however skewed the routing."""
    tiles = -(-M // _WGRAD_TILE) * -(-N // _WGRAD_TILE)   # per expert
    free = max(_compute_units(device) - E * tiles, tiles)
    L = -(-R * tiles // free)
    L = max(256, -(-L // 64) * 64)
    while -(-R // L) + E > 1024:   # the launch takes at most 1024 segments
        L *= 2
    return L


def _gemm_wgrad(a, b, offs, E, dtype, out=None, segs=None):
    """dw[e] (+)= a[rows of e]^T b[rows of e], cut along the rows when the launch would otherwise
    leave most of the chip idle: the segments are the "experts" of one launch with fp32 results,
    which a second kernel adds per expert in a fixed order (reproducible).  `segs` (a dict that
    lives as long as one backward pass) keeps the segments of these `offs` per length, so that the
    three stacks share them."""
    R, M = a.shape
    N = b.shape[1]
    if R == 0 or _wgrad_split(E, M, N, a.device) < 2:
        return ops.gemm_wgrad(a, b, offs, E, dtype, out=out)
    L = _segment_rows(E, M, N, R, a.device)
    held = None if segs is None else segs.get(L)
    if held is None:
        held = ops.segment_offsets_by_length(offs, E, L, R)
        if segs is not None:
            segs[L] = held
    seg, seg_start, S_max = held
    part = ops.gemm_wgrad(a, b, seg, S_max, torch.float32)
    return ops.wgrad_reduce_segments(part, seg_start, E, dtype, out=out)


def _wgrad(a, b, offs, E, wdtype, needed, param, segs=None):
    """One stack's weight gradient.  With `param` given the result goes into `param.grad`
    (added to it when it exists) and None is returned for autograd."""
    if not needed:
        return None
    if param is None:
        return _gemm_wgrad(a, b, offs, E, wdtype, segs=segs)
    held = param.grad
    if held is None:
        param.grad = _gemm_wgrad(a, b, offs, E, param.dtype, segs=segs)
        return None
    if (held.dtype in (torch.float32, torch.bfloat16) and held.is_contiguous()
            and held.shape == (E, a.shape[1], b.shape[1]) and held.device == a.device):
        _gemm_wgrad(a, b, offs, E, held.dtype, out=held, segs=segs)
        return None
    return _gemm_wgrad(a, b, offs, E, wdtype)  # a .grad the kernel cannot add to: autograd sums


def _grad_slot_ok(param, shape, device):
    held = param.grad
    return held is None or (held.dtype in (torch.float32, torch.bfloat16) and held.is_contiguous()
                            and tuple(held.shape) == tuple(shape) and held.device == device)


def _pair_ok(E, I, H, need_w, into, device):
    """Whether the gate and up weight gradients can come out of one launch on the side-by-side
    [dg | du] buffer: both wanted, 256-row tiles of the stacked result do not straddle the halves,
    the launch fills the chip without a row split, and (when the kernel is to add into `.grad`)
    both slots are in the same state."""
    if not (need_w[0] and need_w[1]) or I % _WGRAD_TILE != 0 or _wgrad_split(E, I, H, device) >= 2:
        return False
    p1, p3 = into[0], into[1]
    if p1 is None and p3 is None:
        return True
    if p1 is None or p3 is None:
        return False
    shape = (E, I, H)
    if not (_grad_slot_ok(p1, shape, device) and _grad_slot_ok(p3, shape, device)):
        return False
    g1, g3 = p1.grad, p3.grad
    return (g1 is None) == (g3 is None) and (g1 is None or g1.dtype == g3.dtype) and p1.dtype == p3.dtype


def _gateup(xp, w1b, w3b, offs, train: bool):
    """Gate/up product and SwiGLU of the forward pass: -> (gu, act).  When a backward pass will
    follow, g and u are saved in the library's blocked layout (read by nothing but the SwiGLU
    backward); otherwise they are not written at all and `gu` is None."""
    if train:
        return ops.gemm_gateup_blocked(xp, w1b, w3b, offs)
    return None, ops.gemm_gateup(xp, w1b, w3b, offs, save_gu=False)[2]


def _expert_backward(dyp, xp, gu, act, w1b, w3b, w2b, offs, wdtype, need_w=(True, True, True),
                     into=None, gate_blocks=False):
    """Shared backward of the expert FFN over expert-contiguous rows.  `gu` is the forward's g and
    u in the library's blocked layout (ops.gemm_gateup_blocked).  `need_w` and `into` are per
    stack in the order gate, up, down.  With `gate_blocks` the fifth result holds the per-row block
    sums of <dact, act> (the gate gradients are made from them), else None."""
    E, I, H = w1b.shape
    into = into or (None, None, None)
    part = None
    if dyp.shape[0] > 0 and _pair_ok(E, I, H, need_w, into, dyp.device):
        # dg and du side by side: their two weight gradients are one grouped product
        dgu, part = ops.gemm_dgrad_down_blocked(dyp, w2b, gu, offs, gate_blocks, packed=True)
        dxp = ops.gemm_dgrad_gateup_packed(dgu, w1b, w3b, offs)
        dw2 = _wgrad(dyp, act, offs, E, wdtype, need_w[2], into[2])
        p1, p3 = into[0], into[1]
        if p1 is None:
            dw1, dw3 = ops.gemm_wgrad_pair(dgu, xp, offs, E, wdtype)
        elif p1.grad is None:
            p1.grad, p3.grad = ops.gemm_wgrad_pair(dgu, xp, offs, E, p1.dtype)
            dw1 = dw3 = None
        else:
            ops.gemm_wgrad_pair(dgu, xp, offs, E, p1.grad.dtype, out1=p1.grad, out3=p3.grad)
            dw1 = dw3 = None
        return dxp, dw1, dw3, dw2, part
    dg, du, part = ops.gemm_dgrad_down_blocked(dyp, w2b, gu, offs, gate_blocks)
    dxp = ops.gemm_dgrad_gateup(dg, du, w1b, w3b, offs)
    segs = {}
    dw2 = _wgrad(dyp, act, offs, E, wdtype, need_w[2], into[2], segs)
    dw1 = _wgrad(dg, xp, offs, E, wdtype, need_w[0], into[0], segs)
    dw3 = _wgrad(du, xp, offs, E, wdtype, need_w[1], into[1], segs)
    return dxp, dw1, dw3, dw2, part


class _MoEFFN(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, logits, w1, w3, w2, k, bias, shadows, grad_params):
        T, H = x.shape
        E = logits.shape[1]
        x = _dense(x)
        logits = _dense(logits)
        shadows = shadows or (None, None, None)
        w1b, w3b, w2b = (sh if sh is not None else ops.cast_bf16(_dense(w))
                         for w, sh in zip((w1, w3, w2), shadows))
        ids, gates = ops.router_topk(logits, k, bias)
        counts, offs, pos_to_row, row_to_pos = ops.histogram_scan(ids, E)
        xp = ops.permute_fwd(x, pos_to_row, k, row_to_pos)
        train = any(ctx.needs_input_grad)
        gu, act = _gateup(xp, w1b, w3b, offs, train)
        y = ops.gemm_down(act, w2b, offs)
        out = ops.combine_fwd(y, gates, row_to_pos, T, k, x.dtype)
        if train:  # (y is not kept: the gate gradients come out of the dgrad-down kernel)
            ctx.save_for_backward(xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos,
                                  w1b, w3b, w2b)
        ctx.k, ctx.E = k, E
        ctx.grad_params = grad_params
        ctx.x_dtype, ctx.logits_dtype, ctx.w_dtype = x.dtype, logits.dtype, w1.dtype
        ctx.mark_non_differentiable(ids, gates, counts, offs, pos_to_row, row_to_pos)
        ctx.set_materialize_grads(False)  # no zero tensors made up for the routing outputs
        ctx.out_shape = out.shape
        return out, ids, gates, counts, offs, pos_to_row, row_to_pos

    @staticmethod
    def backward(ctx, dout, *unused):
        _first_order_only()
        xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos, w1b, w3b, w2b = ctx.saved_tensors
        k, E = ctx.k, ctx.E
        if dout is None:
            dout = torch.zeros(ctx.out_shape, dtype=ctx.x_dtype, device=xp.device)
        T = dout.shape[0]
        dout = _dense(dout)
        if dout.dtype not in (torch.bfloat16, torch.float32):
            dout = dout.float()
        dyp, _ = ops.combine_bwd(dout, None, gates, pos_to_row, k, row_to_pos)
        dxp, dw1, dw3, dw2, part = _expert_backward(dyp, xp, gu, act, w1b, w3b, w2b, offs, ctx.w_dtype,
                                                    ctx.needs_input_grad[2:5], ctx.grad_params,
                                                    ctx.needs_input_grad[1] or ctx.needs_input_grad[6])
        dx = ops.permute_bwd(dxp, row_to_pos, T, k, ctx.x_dtype) if ctx.needs_input_grad[0] else None
        dlogits = dbias = None
        if ctx.needs_input_grad[1] or ctx.needs_input_grad[6]:
            dgates = ops.dgates_from_blocks(part, gates, row_to_pos, pos_to_row)
            if ctx.needs_input_grad[6]:  # column sum of the logits' gradient, before any rounding
                dl32 = ops.router_topk_bwd(gates, dgates, ids, T, E, k, torch.float32)
                dbias = dl32.sum(0)
                dlogits = dl32.to(ctx.logits_dtype) if ctx.needs_input_grad[1] else None
            else:
                dlogits = ops.router_topk_bwd(gates, dgates, ids, T, E, k, ctx.logits_dtype)
        return dx, dlogits, dw1, dw3, dw2, None, dbias, None, None


def _forward_only(*tensors) -> bool:
    """Whether a call needs nothing kept for a backward pass: then the whole forward goes to the
    library as one call (`ops.ffn_forward`).  Not while a launch observer is installed: it wants
    to see the launches one by one."""
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        return False
    return ops.launch_observer() is None


def _weights_bf16(w1, w3, w2, shadows):
    shadows = shadows or (None, None, None)
    return [sh if sh is not None else ops.cast_bf16(_dense(w)) for w, sh in zip((w1, w3, w2), shadows)]


def moe_ffn(x: torch.Tensor, logits: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor,
            w2: torch.Tensor, k: int, bias: torch.Tensor | None = None, return_routing: bool = False,
            bf16_weights=None, accumulate_into_grad: bool = False):
    """out[t] = sum_j gate[t,j] * FFN_{e(t,j)}(x[t]).  x [T,H]; logits [T,E]; w1,w3 [E,I,H];
    w2 [E,H,I].  `bias` (fp32 [E]) is added to the logits in fp32 and is part of them from
    there on: both the selection and the softmax over the selected values see logit + bias
    (a per-expert constant in the router, as benchmark config 2 specifies); when it requires a
    gradient it receives the column sum of the logits' gradient (fp32, summed before that gradient
    is rounded to the logits' dtype).
    With `return_routing` also returns a dict of the integer routing tensors and gates.
    `bf16_weights`: bf16 copies of (w1, w3, w2) to compute with (None entries are cast here).
    `accumulate_into_grad`: w1, w3, w2 must be leaf tensors; see the module docstring."""
    if not return_routing and x.shape[0] > 0 and _forward_only(x, logits, w1, w3, w2, bias):
        w1b, w3b, w2b = _weights_bf16(w1, w3, w2, bf16_weights)
        return ops.ffn_forward(_dense(x), _dense(logits), w1b, w3b, w2b, k, bias)
    grad_params = None
    if accumulate_into_grad:
        grad_params = tuple(w if (w.requires_grad and w.is_leaf) else None for w in (w1, w3, w2))
    out, ids, gates, counts, offs, pos_to_row, row_to_pos = _MoEFFN.apply(
        x, logits, w1, w3, w2, k, bias, bf16_weights, grad_params)
    if return_routing:
        return out, {"ids": ids, "gates": gates, "counts": counts, "offs": offs,
                     "pos_to_row": pos_to_row, "row_to_pos": row_to_pos}
    return out


class _MoEFFNf32(torch.autograd.Function):
    """The fp32 path: model/modules/mlp.py:101-167 with fp32 operands and no autocast."""

    @staticmethod
    def forward(ctx, x, logits, w1, w3, w2, k, bias):
        T, H = x.shape
        E = logits.shape[1]
        x, logits = _dense(x), _dense(logits)
        w1, w3, w2 = _dense(w1), _dense(w3), _dense(w2)
        ids, gates = ops.router_topk(logits, k, bias)
        counts, offs, pos_to_row, row_to_pos = ops.histogram_scan(ids, E)
        xp = ops.f32_gather_rows(x, pos_to_row, k)
        g = ops.f32_gemm_rows(xp, w1, offs, True)
        u = ops.f32_gemm_rows(xp, w3, offs, True)
        act = ops.f32_swiglu(g, u)
        y = ops.f32_gemm_rows(act, w2, offs, True)
        out = ops.f32_combine_fwd(y, gates, row_to_pos, T, k)
        if any(ctx.needs_input_grad):
            ctx.save_for_backward(xp, g, u, act, y, gates, ids, offs, pos_to_row, row_to_pos, w1, w3, w2)
        ctx.k, ctx.E = k, E
        ctx.mark_non_differentiable(ids, gates, counts, offs, pos_to_row, row_to_pos)
        ctx.set_materialize_grads(False)
        ctx.out_shape = out.shape
        return out, ids, gates, counts, offs, pos_to_row, row_to_pos

    @staticmethod
    def backward(ctx, dout, *unused):
        _first_order_only()
        xp, g, u, act, y, gates, ids, offs, pos_to_row, row_to_pos, w1, w3, w2 = ctx.saved_tensors
        k, E = ctx.k, ctx.E
        if dout is None:
            dout = torch.zeros(ctx.out_shape, dtype=torch.float32, device=xp.device)
        T = dout.shape[0]
        need = ctx.needs_input_grad
        dyp, dgates = ops.f32_combine_bwd(_dense(dout.float()), y if (need[1] or need[6]) else None, gates,
                                          pos_to_row, k)
        dact = ops.f32_gemm_rows(dyp, w2, offs, False)
        dg, du = ops.f32_swiglu_bwd(dact, g, u)
        dx = None
        if need[0]:
            dxp = ops.f32_gemm_rows(dg, w1, offs, False)
            ops.f32_gemm_rows(du, w3, offs, False, out=dxp)
            dx = ops.f32_permute_bwd(dxp, row_to_pos, T, k)
        dw1 = ops.f32_gemm_wgrad(dg, xp, offs, E) if need[2] else None
        dw3 = ops.f32_gemm_wgrad(du, xp, offs, E) if need[3] else None
        dw2 = ops.f32_gemm_wgrad(dyp, act, offs, E) if need[4] else None
        dlogits = dbias = None
        if need[1] or need[6]:
            dlogits = ops.router_topk_bwd(gates, dgates, ids, T, E, k, torch.float32)
            dbias = dlogits.sum(0) if need[6] else None
            if not need[1]:
                dlogits = None
        return dx, dlogits, dw1, dw3, dw2, None, dbias


def moe_ffn_f32(x: torch.Tensor, logits: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor,
                w2: torch.Tensor, k: int, bias: torch.Tensor | None = None, return_routing: bool = False):
    """`moe_ffn` with every tensor and every product in fp32 (all arguments fp32; H and the FFN
    width multiples of 4).  Routing, counts and the permutation are the same kernels and the same
    bits as in `moe_ffn` given the same logits."""
    for name, t in (("x", x), ("logits", logits), ("w1", w1), ("w3", w3), ("w2", w2)):
        if t.dtype != torch.float32:
            raise TypeError(f"moe_ffn_f32: {name} must be fp32, got {t.dtype}")
    out, ids, gates, counts, offs, pos_to_row, row_to_pos = _MoEFFNf32.apply(x, logits, w1, w3, w2, k, bias)
    if return_routing:
        return out, {"ids": ids, "gates": gates, "counts": counts, "offs": offs,
                     "pos_to_row": pos_to_row, "row_to_pos": row_to_pos}
    return out


_ROUTING_NAMES = ("ids", "gates", "counts", "offs", "pos_to_row", "row_to_pos")


class _PreNormMoE(torch.autograd.Function):
    """Router product, routing, experts and combine as one node, optionally with the caller's
    RMSNorm in front (norm_w) and residual add behind.  Without the norm, xn is x itself
    (rounded to bf16 once if it is fp32)."""

    @staticmethod
    def forward(ctx, x, norm_w, wr, w1, w3, w2, eps, k, bias, shadows, grad_params, add_residual,
                fused_router):
        T, H = x.shape
        E = wr.shape[0]
        x = _dense(x)
        shadows = shadows or (None, None, None)
        w1b, w3b, w2b = (sh if sh is not None else ops.cast_bf16(_dense(w))
                         for w, sh in zip((w1, w3, w2), shadows))
        wrb = wr.detach().to(torch.bfloat16)
        if (fused_router and norm_w is not None and bias is None and T > 0
                and ops.rmsnorm_router_supported(H, E, k)):
            # norm, router product and selection in one kernel: the normalised rows are not read
            # a second time for the router, the logits are selected on before they leave the chip
            nw = norm_w.detach().float().contiguous()
            xn, rstd, logits, ids, gates = ops.rmsnorm_router_fwd(x, nw, eps, _dense(wrb), k)
        else:
            if norm_w is not None:
                nw = norm_w.detach().float().contiguous()
                xn, rstd = ops.rmsnorm_fwd(x, nw, eps)
            else:
                nw = rstd = None
                xn = ops.cast_bf16(x)
            with torch.autocast("cuda", enabled=False):
                logits = xn @ wrb.t()
            ids, gates = ops.router_topk(logits, k, bias)
        counts, offs, pos_to_row, row_to_pos = ops.histogram_scan(ids, E)
        xp = ops.permute_fwd(xn, pos_to_row, k, row_to_pos)
        train = any(ctx.needs_input_grad)
        gu, act = _gateup(xp, w1b, w3b, offs, train)
        y = ops.gemm_down(act, w2b, offs)
        if add_residual:
            out = ops.combine_fwd_residual(y, gates, row_to_pos, x, k)
        else:
            out = ops.combine_fwd(y, gates, row_to_pos, T, k, x.dtype)
        ctx.has_norm = norm_w is not None
        if train:
            ctx.save_for_backward(x if ctx.has_norm else None, nw, rstd, xn, wrb, xp, gu, act, gates, ids,
                                  offs, pos_to_row, row_to_pos, w1b, w3b, w2b)
        ctx.k, ctx.E, ctx.add_residual = k, E, add_residual
        ctx.grad_params = grad_params
        ctx.x_dtype, ctx.x_shape = x.dtype, x.shape
        ctx.nw_dtype = norm_w.dtype if ctx.has_norm else None
        ctx.wr_dtype, ctx.w_dtype = wr.dtype, w1.dtype
        ctx.mark_non_differentiable(ids, gates, counts, offs, pos_to_row, row_to_pos)
        ctx.set_materialize_grads(False)
        return out, logits, ids, gates, counts, offs, pos_to_row, row_to_pos

    @staticmethod
    def backward(ctx, dout, dlogits_ext, *unused):
        _first_order_only()
        (x, nw, rstd, xn, wrb, xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos,
         w1b, w3b, w2b) = ctx.saved_tensors
        k, E = ctx.k, ctx.E
        T = ctx.x_shape[0]
        if dout is None:
            dout = torch.zeros(ctx.x_shape, dtype=ctx.x_dtype, device=xn.device)
        dout = _dense(dout)
        if dout.dtype != ctx.x_dtype:
            dout = dout.to(ctx.x_dtype)
        dyp, _ = ops.combine_bwd(dout, None, gates, pos_to_row, k, row_to_pos)
        dxp, dw1, dw3, dw2, part = _expert_backward(dyp, xp, gu, act, w1b, w3b, w2b, offs, ctx.w_dtype,
                                                    ctx.needs_input_grad[3:6], ctx.grad_params, True)
        dgates = ops.dgates_from_blocks(part, gates, row_to_pos, pos_to_row)
        dbias = None
        if ctx.needs_input_grad[8]:
            # the bias is a per-expert constant added to the logits (in fp32): its gradient is the
            # column sum of the logits' gradient, taken before that is rounded to bf16
            dl32 = ops.router_topk_bwd(gates, dgates, ids, T, E, k, torch.float32)
            if dlogits_ext is not None:
                dl32 = dl32 + dlogits_ext.float()
            dbias = dl32.sum(0)
            dlogits = dl32.to(torch.bfloat16)
        else:
            dlogits = ops.router_topk_bwd(gates, dgates, ids, T, E, k, torch.bfloat16)
            if dlogits_ext is not None:
                dlogits = dlogits + dlogits_ext.to(dlogits.dtype)
        dwr = _router_wgrad(dlogits, xn, ctx.wr_dtype) if ctx.needs_input_grad[2] else None
        dx = dnw = None
        if ctx.needs_input_grad[0] or (ctx.has_norm and ctx.needs_input_grad[1]):
            with torch.autocast("cuda", enabled=False):
                d2 = dlogits @ wrb
            if ctx.has_norm:
                d1 = ops.permute_bwd(dxp, row_to_pos, T, k, ctx.x_dtype)
                dx, dnw = ops.rmsnorm_bwd(x, nw, rstd, d1, d2, dout if ctx.add_residual else None)
                dnw = dnw.to(ctx.nw_dtype) if ctx.needs_input_grad[1] else None
            else:  # the router path's gradient joins the k-row sum in the same pass
                dx = ops.permute_bwd(dxp, row_to_pos, T, k, ctx.x_dtype, addend=d2)
                if ctx.add_residual:
                    dx = dx + dout
            if not ctx.needs_input_grad[0]:
                dx = None
        return dx, dnw, dwr, dw1, dw3, dw2, None, None, dbias, None, None, None, None


def prenorm_moe(x: torch.Tensor, norm_weight: torch.Tensor, router_weight: torch.Tensor,
                w1: torch.Tensor, w3: torch.Tensor, w2: torch.Tensor, k: int, eps: float = 1e-6,
                add_residual: bool = True, bf16_weights=None, accumulate_into_grad: bool = False,
                return_routing: bool = False, fused_router: bool = True):
    """(x + MoE(RMSNorm(x)), router logits) for x [T,H]: model/gpt.py:32-33 with
    model/modules/norm.py:14-19 and model/modules/mlp.py:95-169 in one differentiable call.
    Router logits are bf16 (what the reference produces under its bf16 autocast); the output
    has the dtype of x.  H <= 8192.  `fused_router=False` takes the logits from the library's
    product (bit-identical to what `routed_moe` and `MoE.forward` select on) instead of the fused
    norm+router kernel, whose own summation order can move a bf16 logit by one unit in the last
    place."""
    grad_params = None
    if accumulate_into_grad:
        grad_params = tuple(w if (w.requires_grad and w.is_leaf) else None for w in (w1, w3, w2))
    res = _PreNormMoE.apply(x, norm_weight, router_weight, w1, w3, w2, float(eps), k, None, bf16_weights,
                            grad_params, add_residual, fused_router)
    if return_routing:
        return res[0], res[1], dict(zip(_ROUTING_NAMES, res[2:]))
    return res[0], res[1]


def routed_moe(x: torch.Tensor, router_weight: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor,
               w2: torch.Tensor, k: int, bias: torch.Tensor | None = None, bf16_weights=None,
               accumulate_into_grad: bool = False, return_routing: bool = False):
    """(MoE(x), router logits) for x [T,H]: `router_linear` and `moe_ffn` as one autograd node
    (mlp.py:100-167), so that the two gradient contributions to x (expert path, router path)
    are summed inside the k-row-sum kernel.  The router product is a bf16 library product
    whatever the dtypes (the reference's behaviour under its bf16 autocast); the output has
    the dtype of x.  With `return_routing` a dict of the integer routing tensors and gates is
    returned as a third value."""
    if not return_routing and x.shape[0] > 0 and _forward_only(x, router_weight, w1, w3, w2, bias):
        # nothing to keep for a backward pass: the router product, then the rest in one call
        w1b, w3b, w2b = _weights_bf16(w1, w3, w2, bf16_weights)
        xn = ops.cast_bf16(_dense(x))
        with torch.autocast("cuda", enabled=False):
            logits = xn @ router_weight.detach().to(torch.bfloat16).t()
        return ops.ffn_forward(xn, logits, w1b, w3b, w2b, k, bias, out_dtype=x.dtype), logits
    grad_params = None
    if accumulate_into_grad:
        grad_params = tuple(w if (w.requires_grad and w.is_leaf) else None for w in (w1, w3, w2))
    res = _PreNormMoE.apply(x, None, router_weight, w1, w3, w2, 0.0, k, bias, bf16_weights, grad_params,
                            False, True)
    if return_routing:
        return res[0], res[1], dict(zip(_ROUTING_NAMES, res[2:]))
    return res[0], res[1]


class _ExpertsRows(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rows, ids, w1, w3, w2, grad_params):
        R, H = rows.shape
        E = w1.shape[0]
        rows = _dense(rows)
        ids32 = _dense(ids.to(torch.int32))
        w1b, w3b, w2b = (ops.cast_bf16(_dense(w)) for w in (w1, w3, w2))
        counts, offs, pos_to_row, row_to_pos, bad = ops.histogram_scan(ids32, E, return_bad=True)
        xp = ops.permute_fwd(rows, pos_to_row, 1)
        train = any(ctx.needs_input_grad)
        gu, act = _gateup(xp, w1b, w3b, offs, train)
        y = ops.gemm_down(act, w2b, offs)
        out = ops.combine_fwd(y, None, row_to_pos, R, 1, rows.dtype)
        if train:
            ctx.save_for_backward(xp, gu, act, offs, pos_to_row, row_to_pos, w1b, w3b, w2b)
        ctx.x_dtype, ctx.w_dtype = rows.dtype, w1.dtype
        ctx.grad_params = grad_params
        ctx.mark_non_differentiable(counts, offs, pos_to_row, row_to_pos, bad)
        ctx.set_materialize_grads(False)
        ctx.out_shape = out.shape
        return out, counts, offs, pos_to_row, row_to_pos, bad

    @staticmethod
    def backward(ctx, dout, *unused):
        _first_order_only()
        xp, gu, act, offs, pos_to_row, row_to_pos, w1b, w3b, w2b = ctx.saved_tensors
        if dout is None:
            dout = torch.zeros(ctx.out_shape, dtype=ctx.x_dtype, device=xp.device)
        R = dout.shape[0]
        dout = _dense(dout)
        if dout.dtype not in (torch.bfloat16, torch.float32):
            dout = dout.float()
        dyp, _ = ops.combine_bwd(dout, None, None, pos_to_row, 1)
        dxp, dw1, dw3, dw2, _ = _expert_backward(dyp, xp, gu, act, w1b, w3b, w2b, offs,
                                                 ctx.w_dtype, ctx.needs_input_grad[2:5], ctx.grad_params)
        drows = ops.permute_bwd(dxp, row_to_pos, R, 1, ctx.x_dtype) if ctx.needs_input_grad[0] else None
        return drows, None, dw1, dw3, dw2, None


class _ExpertsRowsF32(torch.autograd.Function):
    @staticmethod
    def forward(ctx, rows, ids, w1, w3, w2):
        R, H = rows.shape
        E = w1.shape[0]
        rows, w1, w3, w2 = _dense(rows), _dense(w1), _dense(w3), _dense(w2)
        ids32 = _dense(ids.to(torch.int32))
        counts, offs, pos_to_row, row_to_pos, bad = ops.histogram_scan(ids32, E, return_bad=True)
        xp = ops.f32_gather_rows(rows, pos_to_row, 1)
        g = ops.f32_gemm_rows(xp, w1, offs, True)
        u = ops.f32_gemm_rows(xp, w3, offs, True)
        act = ops.f32_swiglu(g, u)
        y = ops.f32_gemm_rows(act, w2, offs, True)
        out = ops.f32_combine_fwd(y, None, row_to_pos, R, 1)
        if any(ctx.needs_input_grad):
            ctx.save_for_backward(xp, g, u, act, offs, pos_to_row, row_to_pos, w1, w3, w2)
        ctx.mark_non_differentiable(counts, offs, pos_to_row, row_to_pos, bad)
        ctx.set_materialize_grads(False)
        ctx.out_shape = out.shape
        return out, counts, offs, pos_to_row, row_to_pos, bad

    @staticmethod
    def backward(ctx, dout, *unused):
        _first_order_only()
        xp, g, u, act, offs, pos_to_row, row_to_pos, w1, w3, w2 = ctx.saved_tensors
        if dout is None:
            dout = torch.zeros(ctx.out_shape, dtype=torch.float32, device=xp.device)
        R, E = dout.shape[0], w1.shape[0]
        need = ctx.needs_input_grad
        dyp, _ = ops.f32_combine_bwd(_dense(dout.float()), None, None, pos_to_row, 1)
        dg, du = ops.f32_swiglu_bwd(ops.f32_gemm_rows(dyp, w2, offs, False), g, u)
        drows = None
        if need[0]:
            dxp = ops.f32_gemm_rows(dg, w1, offs, False)
            ops.f32_gemm_rows(du, w3, offs, False, out=dxp)
            drows = ops.f32_permute_bwd(dxp, row_to_pos, R, 1)
        dw1 = ops.f32_gemm_wgrad(dg, xp, offs, E) if need[2] else None
        dw3 = ops.f32_gemm_wgrad(du, xp, offs, E) if need[3] else None
        dw2 = ops.f32_gemm_wgrad(dyp, act, offs, E) if need[4] else None
        return drows, None, dw1, dw3, dw2


def experts_rows_f32(rows: torch.Tensor, ids: torch.Tensor, w1, w3, w2, return_routing: bool = False,
                     check_ids: bool = False):
    """`experts_rows` with every tensor and every product in fp32 (rows and weights fp32)."""
    for name, t in (("rows", rows), ("w1", w1), ("w3", w3), ("w2", w2)):
        if t.dtype != torch.float32:
            raise TypeError(f"experts_rows_f32: {name} must be fp32, got {t.dtype}")
    out, counts, offs, pos_to_row, row_to_pos, bad = _ExpertsRowsF32.apply(rows, ids, w1, w3, w2)
    if check_ids:
        n = int(bad.item())
        if n:
            raise ValueError(f"experts_rows_f32: {n} of {ids.numel()} expert ids lie outside [0, {w1.shape[0]})")
    if return_routing:
        return out, {"counts": counts, "offs": offs, "pos_to_row": pos_to_row, "row_to_pos": row_to_pos,
                     "bad_ids": bad}
    return out


def experts_rows(rows: torch.Tensor, ids: torch.Tensor, w1, w3, w2, return_routing: bool = False,
                 accumulate_into_grad: bool = False, check_ids: bool = False):
    """One rank's local expert share: rows [R,H] already dispatched to this rank, ids [R]
    local expert index of each row -> FFN output rows in the same (arrival) order.

    ids must lie in [0, E).  The dispatch kernels count the ids that do not (and treat such a
    row as belonging to the nearest valid expert, so nothing reads out of bounds); the count is
    a device tensor, `bad_ids` in the routing dict, so the hot path never waits for it.  With
    `check_ids` the call synchronises and raises ValueError if the count is not zero."""
    grad_params = None
    if accumulate_into_grad:
        grad_params = tuple(w if (w.requires_grad and w.is_leaf) else None for w in (w1, w3, w2))
    out, counts, offs, pos_to_row, row_to_pos, bad = _ExpertsRows.apply(rows, ids, w1, w3, w2, grad_params)
    if check_ids:
        n = int(bad.item())
        if n:
            raise ValueError(f"experts_rows: {n} of {ids.numel()} expert ids lie outside [0, {w1.shape[0]})")
    if return_routing:
        return out, {"counts": counts, "offs": offs, "pos_to_row": pos_to_row, "row_to_pos": row_to_pos,
                     "bad_ids": bad}
    return out
