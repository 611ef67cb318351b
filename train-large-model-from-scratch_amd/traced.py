"""The layer body as `torch.library` operators, for callers that compile the model.

The reference's trainer wraps the model in `torch.compile` when asked to
(training/trainer.py:130-131) and hides its own opaque step from the tracer with
`torch._dynamo.disable` (distributed/expert_parallel/comm.py:42), which splits the graph in
every MoE layer.  The two operators below, `moe_gfx950::ffn_fwd` and `moe_gfx950::ffn_bwd`,
carry shape-and-dtype-only ("fake") implementations and an autograd formula, so the tracer
can keep `MoE.forward` inside one graph, forward and backward: the kernels stay opaque calls,
everything around them is traced.  `MoE.forward` takes this route only while it is being
traced; eager calls use `functional.moe_ffn` (same kernels, plus the cached weight copies).

A second pair, `moe_gfx950::routed_fwd` / `routed_bwd`, has the router product inside (the traced
counterpart of `functional.routed_moe`, what the module's eager call runs under bf16 autocast), and
a third, `moe_gfx950::ffn_f32_fwd` / `ffn_f32_bwd` at the end of the file, does the same for the
fp32 path (`functional.moe_ffn_f32`).

Semantics of the first pair are those of `functional.moe_ffn`: bf16 matrix-core compute with fp32
accumulation, output and input gradient in the dtype of x, weight gradients in the dtype of
the weights.  fp32 weights are rounded to bf16 inside the forward operator (three casts per
call, what the reference pays too, mlp.py:154-157 under autocast) and the copies are handed to
the backward operator.
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import ops
from .functional import _expert_backward, _router_wgrad

_BF16 = torch.bfloat16


def _empty(ref: Tensor, dtype=_BF16) -> Tensor:
    return torch.empty(0, dtype=dtype, device=ref.device)


def gu_blocked_bytes(R, E: int, I: int):
    """Size of ops.gemm_gateup_blocked's buffer, as arithmetic a symbolic row count passes through:
    moe_gu_blocked_bytes (4 KB per 32 x 32 block of ceil(R/256) + E row tiles of 256 rows), with
    the wrapper's floor of 16 bytes."""
    return (((R + 255) // 256 + E) * 8 * ((I + 31) // 32) * 4096) if R > 0 else 16


@torch.library.custom_op("moe_gfx950::ffn_fwd", mutates_args=(), device_types="cuda")
def ffn_fwd(x: Tensor, logits: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, k: int,
            train: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor,
                                  Tensor, Tensor, Tensor, Tensor]:
    """-> out, ids, gates, offs, pos_to_row, row_to_pos, xp, gu, act, w1b, w3b, w2b.
    `gu` holds g and u in the library's blocked layout (an opaque uint8 buffer that only the
    backward operator reads; empty without `train`); a weight that already is bf16 has an empty
    copy."""
    T, H = x.shape
    E = logits.shape[1]
    x, logits = ops.dense(x), ops.dense(logits)
    wb = [ops.dense(w) if w.dtype == _BF16 else ops.cast_bf16(ops.dense(w)) for w in (w1, w3, w2)]
    ids, gates = ops.router_topk(logits, k, None)
    _, offs, pos_to_row, row_to_pos = ops.histogram_scan(ids, E)
    xp = ops.permute_fwd(x, pos_to_row, k, row_to_pos)
    if train:
        gu, act = ops.gemm_gateup_blocked(xp, wb[0], wb[1], offs)
    else:
        gu, act = _empty(x, torch.uint8), ops.gemm_gateup(xp, wb[0], wb[1], offs, save_gu=False)[2]
    y = ops.gemm_down(act, wb[2], offs)
    out = ops.combine_fwd(y, gates, row_to_pos, T, k, x.dtype)
    copies = [b if w.dtype != _BF16 else _empty(x) for w, b in zip((w1, w3, w2), wb)]
    return (out, ids, gates, offs, pos_to_row, row_to_pos, xp, gu, act, *copies)


@ffn_fwd.register_fake
def _(x, logits, w1, w3, w2, k, train):
    T, H = x.shape
    E, I = logits.shape[1], w1.shape[1]
    R = T * k
    i32 = lambda *s: x.new_empty(s, dtype=torch.int32)
    b16 = lambda *s: x.new_empty(s, dtype=_BF16)
    gu_bytes = gu_blocked_bytes(R, E, I) if train else 0
    copies = [b16(*w.shape) if w.dtype != _BF16 else b16(0) for w in (w1, w3, w2)]
    return (x.new_empty(T, H), i32(R), x.new_empty(R, dtype=torch.float32), i32(E + 1), i32(R), i32(R),
            b16(R, H), x.new_empty(gu_bytes, dtype=torch.uint8), b16(R, I), *copies)


@torch.library.custom_op("moe_gfx950::ffn_bwd", mutates_args=(), device_types="cuda")
def ffn_bwd(dout: Tensor, xp: Tensor, gu: Tensor, act: Tensor, gates: Tensor,
            ids: Tensor, offs: Tensor, pos_to_row: Tensor, row_to_pos: Tensor, w1b: Tensor,
            w3b: Tensor, w2b: Tensor, k: int, x_is_f32: bool, logits_is_f32: bool,
            w_is_f32: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> dx, dlogits, dw1, dw3, dw2.  The kernels of the eager backward pass
    (`functional._expert_backward`)."""
    T = dout.shape[0]
    E = offs.numel() - 1
    f32 = torch.float32
    dout = ops.dense(dout)
    if dout.dtype not in (_BF16, f32):
        dout = dout.float()
    dyp, _ = ops.combine_bwd(dout, None, gates, pos_to_row, k, row_to_pos)
    wdt = f32 if w_is_f32 else _BF16
    dxp, dw1, dw3, dw2, part = _expert_backward(dyp, xp, gu, act, w1b, w3b, w2b, offs, wdt, gate_blocks=True)
    dgates = ops.dgates_from_blocks(part, gates, row_to_pos, pos_to_row)
    dx = ops.permute_bwd(dxp, row_to_pos, T, k, f32 if x_is_f32 else _BF16)
    dlogits = ops.router_topk_bwd(gates, dgates, ids, T, E, k, f32 if logits_is_f32 else _BF16)
    return dx, dlogits, dw1, dw3, dw2


@ffn_bwd.register_fake
def _(dout, xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos, w1b, w3b, w2b, k, x_is_f32,
      logits_is_f32, w_is_f32):
    T, H = dout.shape
    E = offs.shape[0] - 1
    f32 = torch.float32
    wdt = f32 if w_is_f32 else _BF16
    return (dout.new_empty(T, H, dtype=f32 if x_is_f32 else _BF16),
            dout.new_empty(T, E, dtype=f32 if logits_is_f32 else _BF16),
            dout.new_empty(w1b.shape, dtype=wdt), dout.new_empty(w3b.shape, dtype=wdt),
            dout.new_empty(w2b.shape, dtype=wdt))


def _setup_context(ctx, inputs, output):
    x, logits, w1, w3, w2, k, train = inputs
    out, ids, gates, offs, pos_to_row, row_to_pos, xp, gu, act, w1b, w3b, w2b = output
    # the bf16 operands: the copy made in the forward, or the weight itself
    wb = [w if w.dtype == _BF16 else b for w, b in zip((w1, w3, w2), (w1b, w3b, w2b))]
    ctx.save_for_backward(xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos, *wb)
    ctx.k, ctx.train = k, train
    ctx.flags = (x.dtype == torch.float32, logits.dtype == torch.float32, w1.dtype == torch.float32)


def _backward(ctx, dout, *unused):
    if not ctx.train:
        raise RuntimeError("moe_gfx950::ffn_fwd was called with train=False: nothing was saved for backward")
    xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos, w1b, w3b, w2b = ctx.saved_tensors
    dx, dlogits, dw1, dw3, dw2 = ffn_bwd(dout, xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos,
                                         w1b, w3b, w2b, ctx.k, *ctx.flags)
    return dx, dlogits, dw1, dw3, dw2, None, None


ffn_fwd.register_autograd(_backward, setup_context=_setup_context)


def moe_ffn(x: Tensor, logits: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, k: int) -> Tensor:
    """Traceable counterpart of `functional.moe_ffn(x, logits, w1, w3, w2, k)`."""
    train = torch.is_grad_enabled() and any(t.requires_grad for t in (x, logits, w1, w3, w2))
    return ffn_fwd(x, logits, w1, w3, w2, k, train)[0]


# ---- router product + layer body as one pair (functional.routed_moe) ------------------------------

@torch.library.custom_op("moe_gfx950::routed_fwd", mutates_args=(), device_types="cuda")
def routed_fwd(x: Tensor, wr: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, k: int,
               train: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor,
                                     Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> out, logits, ids, gates, offs, pos_to_row, row_to_pos, xn, wrb, xp, gu, act, w1b, w3b, w2b.
    The forward of `functional.routed_moe`: the router logits are a bf16 library product on the
    bf16 rows (`xn`) and the bf16 router weight (`wrb`); the rest as in `ffn_fwd`.  A bf16 copy of
    a tensor that already is bf16 is empty; without `train` so are xn, wrb, xp, gu and act."""
    T, H = x.shape
    E = wr.shape[0]
    x = ops.dense(x)
    wb = [ops.cast_bf16(ops.dense(w)) for w in (w1, w3, w2)]
    xn = ops.cast_bf16(x)
    wrb = ops.dense(wr.detach().to(_BF16))
    with torch.autocast("cuda", enabled=False):
        logits = xn @ wrb.t()
    ids, gates = ops.router_topk(logits, k, None)
    _, offs, pos_to_row, row_to_pos = ops.histogram_scan(ids, E)
    xp = ops.permute_fwd(xn, pos_to_row, k, row_to_pos)
    if train:
        gu, act = ops.gemm_gateup_blocked(xp, wb[0], wb[1], offs)
    else:
        gu, act = _empty(x, torch.uint8), ops.gemm_gateup(xp, wb[0], wb[1], offs, save_gu=False)[2]
    y = ops.gemm_down(act, wb[2], offs)
    out = ops.combine_fwd(y, gates, row_to_pos, T, k, x.dtype)
    copies = [b if w.dtype != _BF16 else _empty(x) for w, b in zip((w1, w3, w2), wb)]
    if not train:
        return (out, logits, ids, gates, offs, pos_to_row, row_to_pos, _empty(x), _empty(x), _empty(x), gu,
                _empty(x), *copies)
    return (out, logits, ids, gates, offs, pos_to_row, row_to_pos, xn if x.dtype != _BF16 else _empty(x),
            wrb if wr.dtype != _BF16 else _empty(x), xp, gu, act, *copies)


@routed_fwd.register_fake
def _(x, wr, w1, w3, w2, k, train):
    T, H = x.shape
    E, I = wr.shape[0], w1.shape[1]
    R = T * k
    i32 = lambda *s: x.new_empty(s, dtype=torch.int32)
    b16 = lambda *s: x.new_empty(s, dtype=_BF16)
    copies = [b16(*w.shape) if w.dtype != _BF16 else b16(0) for w in (w1, w3, w2)]
    xn = b16(T, H) if (train and x.dtype != _BF16) else b16(0)
    wrb = b16(E, H) if (train and wr.dtype != _BF16) else b16(0)
    gu = x.new_empty(gu_blocked_bytes(R, E, I) if train else 0, dtype=torch.uint8)
    return (x.new_empty(T, H), b16(T, E), i32(R), x.new_empty(R, dtype=torch.float32), i32(E + 1), i32(R),
            i32(R), xn, wrb, b16(R, H) if train else b16(0), gu, b16(R, I) if train else b16(0), *copies)


@torch.library.custom_op("moe_gfx950::routed_bwd", mutates_args=(), device_types="cuda")
def routed_bwd(dout: Tensor, dlogits_ext: Tensor | None, xn: Tensor, wrb: Tensor, xp: Tensor, gu: Tensor,
               act: Tensor, gates: Tensor, ids: Tensor, offs: Tensor, pos_to_row: Tensor,
               row_to_pos: Tensor, w1b: Tensor, w3b: Tensor, w2b: Tensor, k: int, x_is_f32: bool,
               wr_is_f32: bool, w_is_f32: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> dx, dwr, dw1, dw3, dw2.  The backward of `functional.routed_moe`: `dlogits_ext` is the
    gradient that reaches the returned logits from outside (an auxiliary loss) or None; the router
    path's input gradient joins the k-row sum inside the permute-backward kernel."""
    T = dout.shape[0]
    E = offs.numel() - 1
    f32 = torch.float32
    xdt = f32 if x_is_f32 else _BF16
    dout = ops.dense(dout)
    if dout.dtype != xdt:
        dout = dout.to(xdt)
    dyp, _ = ops.combine_bwd(dout, None, gates, pos_to_row, k, row_to_pos)
    dxp, dw1, dw3, dw2, part = _expert_backward(dyp, xp, gu, act, w1b, w3b, w2b, offs,
                                                f32 if w_is_f32 else _BF16, gate_blocks=True)
    dgates = ops.dgates_from_blocks(part, gates, row_to_pos, pos_to_row)
    dlogits = ops.router_topk_bwd(gates, dgates, ids, T, E, k, _BF16)
    if dlogits_ext is not None:
        dlogits = dlogits + dlogits_ext.to(_BF16)
    dwr = _router_wgrad(dlogits, xn, f32 if wr_is_f32 else _BF16)
    with torch.autocast("cuda", enabled=False):
        d2 = dlogits @ wrb
    dx = ops.permute_bwd(dxp, row_to_pos, T, k, xdt, addend=d2)
    return dx, dwr, dw1, dw3, dw2


@routed_bwd.register_fake
def _(dout, dlogits_ext, xn, wrb, xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos, w1b, w3b, w2b, k,
      x_is_f32, wr_is_f32, w_is_f32):
    T, H = dout.shape
    f32 = torch.float32
    wdt = f32 if w_is_f32 else _BF16
    return (dout.new_empty(T, H, dtype=f32 if x_is_f32 else _BF16),
            dout.new_empty(wrb.shape, dtype=f32 if wr_is_f32 else _BF16),
            dout.new_empty(w1b.shape, dtype=wdt), dout.new_empty(w3b.shape, dtype=wdt),
            dout.new_empty(w2b.shape, dtype=wdt))


def _setup_context_routed(ctx, inputs, output):
    x, wr, w1, w3, w2, k, train = inputs
    (out, logits, ids, gates, offs, pos_to_row, row_to_pos, xn, wrb, xp, gu, act, w1b, w3b, w2b) = output
    wb = [w if w.dtype == _BF16 else b for w, b in zip((w1, w3, w2), (w1b, w3b, w2b))]
    ctx.save_for_backward(x if x.dtype == _BF16 else xn, wr if wr.dtype == _BF16 else wrb, xp, gu, act, gates,
                          ids, offs, pos_to_row, row_to_pos, *wb)
    ctx.k, ctx.train = k, train
    ctx.x_shape, ctx.x_dtype = x.shape, x.dtype
    ctx.flags = (x.dtype == torch.float32, wr.dtype == torch.float32, w1.dtype == torch.float32)
    ctx.set_materialize_grads(False)  # no zero tensor made up for logits nobody differentiates


def _backward_routed(ctx, dout, dlogits_ext, *unused):
    if not ctx.train:
        raise RuntimeError("moe_gfx950::routed_fwd was called with train=False: nothing was saved for backward")
    xn, wrb, xp, gu, act, gates, ids, offs, pos_to_row, row_to_pos, w1b, w3b, w2b = ctx.saved_tensors
    if dout is None:
        dout = torch.zeros(ctx.x_shape, dtype=ctx.x_dtype, device=xp.device)
    dx, dwr, dw1, dw3, dw2 = routed_bwd(dout, dlogits_ext, xn, wrb, xp, gu, act, gates, ids, offs, pos_to_row,
                                        row_to_pos, w1b, w3b, w2b, ctx.k, *ctx.flags)
    return dx, dwr, dw1, dw3, dw2, None, None


routed_fwd.register_autograd(_backward_routed, setup_context=_setup_context_routed)


def routed_moe(x: Tensor, wr: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, k: int) -> tuple[Tensor, Tensor]:
    """Traceable counterpart of `functional.routed_moe(x, wr, w1, w3, w2, k)` -> (out, logits)."""
    train = torch.is_grad_enabled() and any(t.requires_grad for t in (x, wr, w1, w3, w2))
    res = routed_fwd(x, wr, w1, w3, w2, k, train)
    return res[0], res[1]


# ---- the same pair of operators for the fp32 path (functional.moe_ffn_f32) ------------------------

@torch.library.custom_op("moe_gfx950::ffn_f32_fwd", mutates_args=(), device_types="cuda")
def ffn_f32_fwd(x: Tensor, logits: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, k: int,
                train: bool) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor,
                                      Tensor, Tensor, Tensor]:
    """-> out, ids, gates, offs, pos_to_row, row_to_pos, xp, g, u, act, y (all floating point
    tensors fp32).  Without `train` xp, g, u, act and y are empty."""
    T, H = x.shape
    E = logits.shape[1]
    x, logits = ops.dense(x), ops.dense(logits)
    w1, w3, w2 = ops.dense(w1), ops.dense(w3), ops.dense(w2)
    ids, gates = ops.router_topk(logits, k, None)
    _, offs, pos_to_row, row_to_pos = ops.histogram_scan(ids, E)
    xp = ops.f32_gather_rows(x, pos_to_row, k)
    g = ops.f32_gemm_rows(xp, w1, offs, True)
    u = ops.f32_gemm_rows(xp, w3, offs, True)
    act = ops.f32_swiglu(g, u)
    y = ops.f32_gemm_rows(act, w2, offs, True)
    out = ops.f32_combine_fwd(y, gates, row_to_pos, T, k)
    if not train:
        e = _empty(x, torch.float32)
        xp, g, u, act, y = e, e.clone(), e.clone(), e.clone(), e.clone()
    return out, ids, gates, offs, pos_to_row, row_to_pos, xp, g, u, act, y


@ffn_f32_fwd.register_fake
def _(x, logits, w1, w3, w2, k, train):
    T, H = x.shape
    E, I = logits.shape[1], w1.shape[1]
    R = T * k
    i32 = lambda *s: x.new_empty(s, dtype=torch.int32)
    f32 = lambda *s: x.new_empty(s, dtype=torch.float32)
    rh, ri = ((R, H), (R, I)) if train else ((0,), (0,))
    return (f32(T, H), i32(R), f32(R), i32(E + 1), i32(R), i32(R), f32(*rh), f32(*ri), f32(*ri), f32(*ri),
            f32(*rh))


@torch.library.custom_op("moe_gfx950::ffn_f32_bwd", mutates_args=(), device_types="cuda")
def ffn_f32_bwd(dout: Tensor, xp: Tensor, g: Tensor, u: Tensor, act: Tensor, y: Tensor, gates: Tensor,
                ids: Tensor, offs: Tensor, pos_to_row: Tensor, row_to_pos: Tensor, w1: Tensor, w3: Tensor,
                w2: Tensor, k: int) -> tuple[Tensor, Tensor, Tensor, Tensor, Tensor]:
    """-> dx, dlogits, dw1, dw3, dw2 (fp32)."""
    T = dout.shape[0]
    E = offs.numel() - 1
    w1, w3, w2 = ops.dense(w1), ops.dense(w3), ops.dense(w2)
    dyp, dgates = ops.f32_combine_bwd(ops.dense(dout.float()), y, gates, pos_to_row, k)
    dg, du = ops.f32_swiglu_bwd(ops.f32_gemm_rows(dyp, w2, offs, False), g, u)
    dxp = ops.f32_gemm_rows(dg, w1, offs, False)
    ops.f32_gemm_rows(du, w3, offs, False, out=dxp)
    dx = ops.f32_permute_bwd(dxp, row_to_pos, T, k)
    dw1 = ops.f32_gemm_wgrad(dg, xp, offs, E)
    dw3 = ops.f32_gemm_wgrad(du, xp, offs, E)
    dw2 = ops.f32_gemm_wgrad(dyp, act, offs, E)
    dlogits = ops.router_topk_bwd(gates, dgates, ids, T, E, k, torch.float32)
    return dx, dlogits, dw1, dw3, dw2


@ffn_f32_bwd.register_fake
def _(dout, xp, g, u, act, y, gates, ids, offs, pos_to_row, row_to_pos, w1, w3, w2, k):
    T, H = dout.shape
    E = offs.shape[0] - 1
    f32 = lambda *s: dout.new_empty(s, dtype=torch.float32)
    return f32(T, H), f32(T, E), f32(*w1.shape), f32(*w3.shape), f32(*w2.shape)


def _setup_context_f32(ctx, inputs, output):
    x, logits, w1, w3, w2, k, train = inputs
    out, ids, gates, offs, pos_to_row, row_to_pos, xp, g, u, act, y = output
    ctx.save_for_backward(xp, g, u, act, y, gates, ids, offs, pos_to_row, row_to_pos, w1, w3, w2)
    ctx.k, ctx.train = k, train


def _backward_f32(ctx, dout, *unused):
    if not ctx.train:
        raise RuntimeError("moe_gfx950::ffn_f32_fwd was called with train=False: nothing was saved for backward")
    xp, g, u, act, y, gates, ids, offs, pos_to_row, row_to_pos, w1, w3, w2 = ctx.saved_tensors
    dx, dlogits, dw1, dw3, dw2 = ffn_f32_bwd(dout, xp, g, u, act, y, gates, ids, offs, pos_to_row, row_to_pos,
                                             w1, w3, w2, ctx.k)
    return dx, dlogits, dw1, dw3, dw2, None, None


ffn_f32_fwd.register_autograd(_backward_f32, setup_context=_setup_context_f32)


def moe_ffn_f32(x: Tensor, logits: Tensor, w1: Tensor, w3: Tensor, w2: Tensor, k: int) -> Tensor:
    """Traceable counterpart of `functional.moe_ffn_f32(x, logits, w1, w3, w2, k)`."""
    train = torch.is_grad_enabled() and any(t.requires_grad for t in (x, logits, w1, w3, w2))
    return ffn_f32_fwd(x, logits, w1, w3, w2, k, train)[0]
