"""CPU oracle for the MoE expert path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain numpy (integer parts) and plain torch CPU ops (floating
point parts), what the reference's `MoE.forward` (model/modules/mlp.py:95-169) and its
autograd backward compute.  It is the checker the HIP path is compared against; nothing in
the shipped package may import it (only tests, the smoke check and the benchmark's CPU
baseline leg do).

Conventions
-----------
T tokens, H hidden, E experts, k experts per token, R = T*k routed rows, I expert FFN width.
Flat routed row r = t*k + j (token-major, slot j = rank of the selected logit), exactly the
flattening of mlp.py:102-104.  "pos" is a position in the expert-contiguous order.

Canonical choices where the reference leaves the result to the library (its `topk` tie
order and the order of a non-stable `argsort` are unspecified, mlp.py:101,107,123):
  * top-k: order experts by (logit descending, expert index ascending), take the first k;
  * permutation: stable sort of the flat rows by expert id.
The layer output does not depend on either choice, the integer tensors do.

Pin status of every function is listed next to it ("pinned by") and tested in
tests/test_oracle.py.  The reference has no tests, fixtures or golden vectors of its own,
so none of these pins comes from reference-held data: each is a closed form, an invariant,
a brute force on tiny inputs, or an independent library routine.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- routing
def router_logits(x2d: torch.Tensor, wr: torch.Tensor, bias: torch.Tensor | None = None,
                  logits_dtype: torch.dtype | None = None) -> torch.Tensor:
    """gate_logits = router(x)   (mlp.py:100; `nn.Linear(H, E, bias=False)`, mlp.py:65).

    `bias` is not part of the reference module; the skewed-load benchmark config adds a
    per-expert constant to the logits before selection.  `logits_dtype` reproduces the
    autocast behaviour (the linear's output is bf16 there).
    pinned by: torch.nn.functional.linear is the library routine itself.
    """
    out = F.linear(x2d, wr)
    if bias is not None:
        out = out + bias
    if logits_dtype is not None:
        out = out.to(logits_dtype)
    return out


def topk_select(logits: torch.Tensor, k: int) -> tuple[np.ndarray, torch.Tensor]:
    """Canonical top-k of mlp.py:101: ids[T,k] int64 and the selected logits [T,k].

    Slots are in descending-logit order (torch.topk's `sorted=True` default); equal
    logits are ordered by ascending expert index; a NaN ranks above every number, as it
    does for torch.topk.
    pinned by: brute-force insertion on tiny inputs, equality with torch.topk on rows
    without ties (rows with one NaN, with +-inf included), selected-value multiset equality
    on rows with ties.
    """
    lg = logits.detach().to(torch.float64).cpu().numpy()  # exact for bf16/fp32 values
    T, E = lg.shape
    assert 0 < k <= E
    eidx = np.broadcast_to(np.arange(E), (T, E))
    nan = np.isnan(lg)
    # lexsort: last key is primary.  NaNs first, then -logit (descending), then the index.
    order = np.lexsort((eidx, np.where(nan, 0.0, -lg), ~nan), axis=-1)[:, :k].astype(np.int64)
    sel = torch.gather(logits, 1, torch.from_numpy(order).to(logits.device))
    return order, sel


def gates_from_selected(sel_logits: torch.Tensor) -> torch.Tensor:
    """weights = softmax(top-k logits) in fp32 (mlp.py:102; softmax runs in fp32 under
    autocast).  pinned by: library softmax; invariants sum==1, k==1 -> 1, and equality
    with softmax-over-all-experts -> top-k -> renormalise."""
    return F.softmax(sel_logits.to(torch.float32) if sel_logits.dtype != torch.float64
                     else sel_logits, dim=-1)


def counts_offsets(ids_flat: np.ndarray, num_experts: int) -> tuple[np.ndarray, np.ndarray]:
    """counts = bincount(ids, minlength=E); offs = cumsum(counts) (mlp.py:126-127).

    Returns (counts int64 [E], starts int32 [E+1]) with starts[0] = 0 and
    starts[1:] equal to the reference's inclusive `offs`.
    pinned by: np.bincount / np.cumsum are the library routines; invariants in tests.
    """
    counts = np.bincount(ids_flat, minlength=num_experts).astype(np.int64)
    starts = np.zeros(num_experts + 1, dtype=np.int32)
    starts[1:] = np.cumsum(counts).astype(np.int32)
    return counts, starts


def stable_permutation(ids_flat: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """The composed sort of mlp.py:107 and :123 on one rank, made canonical.

    Returns (pos_to_row, row_to_pos): pos_to_row[pos] is the flat routed row that lands at
    expert-contiguous position pos (== `global_sort_idx[local_sort_idx]` when the library
    sort is stable); row_to_pos is its inverse (== the composition of the two
    `argsort(sort_idx)` of mlp.py:160,163).
    pinned by: np.argsort(kind="stable") is the library routine; brute-force counting
    sort on tiny inputs; bijection / monotonicity invariants.
    """
    pos_to_row = np.argsort(ids_flat, kind="stable").astype(np.int64)
    row_to_pos = np.empty_like(pos_to_row)
    row_to_pos[pos_to_row] = np.arange(len(ids_flat), dtype=np.int64)
    return pos_to_row, row_to_pos


# --------------------------------------------------------------------------- experts
def _maybe_round(t: torch.Tensor, emulate_bf16: bool) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype) if emulate_bf16 else t


def expert_ffn_rows(xp: torch.Tensor, starts: np.ndarray, w1: torch.Tensor, w3: torch.Tensor,
                    w2: torch.Tensor, emulate_bf16: bool = False) -> dict[str, torch.Tensor]:
    """Per-expert loop of `down(silu(gate(x)) * up(x))` over expert-contiguous rows.

    One expert is `MLP.forward` (mlp.py:43-44); the reference batches the same products as
    three padded `bmm`s with W^T (mlp.py:154-157).  An expert with zero rows contributes
    nothing.  With `emulate_bf16` the stored intermediates g, u, act, y are rounded to
    bf16 where the device pipeline stores bf16 (the math stays in the input dtype).
    pinned by: E=1 reduces to the dense MLP formula; equality with the literal padded-bmm
    restatement below; torch's own grouped_mm on CPU where available.
    """
    R = xp.shape[0]
    I = w1.shape[1]
    Hh = w2.shape[1]
    g = xp.new_zeros(R, I)
    u = xp.new_zeros(R, I)
    act = xp.new_zeros(R, I)
    y = xp.new_zeros(R, Hh)
    for e in range(w1.shape[0]):
        a, b = int(starts[e]), int(starts[e + 1])
        if a == b:
            continue
        ge = F.linear(xp[a:b], w1[e])
        ue = F.linear(xp[a:b], w3[e])
        ae = _maybe_round(F.silu(ge) * ue, emulate_bf16)
        g[a:b] = _maybe_round(ge, emulate_bf16)
        u[a:b] = _maybe_round(ue, emulate_bf16)
        act[a:b] = ae
        y[a:b] = _maybe_round(F.linear(ae, w2[e]), emulate_bf16)
    return {"g": g, "u": u, "act": act, "y": y}


def combine_rows(y: torch.Tensor, gates_flat: torch.Tensor, row_to_pos: np.ndarray,
                 T: int, k: int) -> torch.Tensor:
    """out[t] = sum_j gate[t,j] * y[row_to_pos[t*k+j]], summed in slot order j = 0..k-1
    (mlp.py:160-167: un-sort, scale by the gate, `.view(T, k, D).sum(1)`).
    pinned by: k=1 with gate 1 is a pure un-permute; linearity in y and in gates."""
    rows = y[torch.from_numpy(row_to_pos)]
    rows = rows * gates_flat.to(rows.dtype).unsqueeze(-1)
    return rows.view(T, k, -1).sum(dim=1)


# --------------------------------------------------------------------------- whole layer
def moe_forward(x: torch.Tensor, wr: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor,
                w2: torch.Tensor, k: int, bias: torch.Tensor | None = None,
                logits: torch.Tensor | None = None, logits_dtype: torch.dtype | None = None,
                compute_dtype: torch.dtype = torch.float32,
                emulate_bf16: bool = False) -> dict:
    """Forward of mlp.py:95-169 on one rank (the all-to-alls are identity copies there).

    x [T,H] (or [B,T,H]); wr [E,H]; w1,w3 [E,I,H]; w2 [E,H,I].  Inputs may be bf16; the
    math runs in `compute_dtype` on exactly those values.  `logits` overrides the router
    product so that routing can be compared on bit-identical logits.
    Returns every intermediate by name.
    """
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).to(compute_dtype)
    T, H = x2.shape
    E = wr.shape[0]
    if logits is None:
        logits = router_logits(x2, wr.to(compute_dtype),
                               None if bias is None else bias.to(compute_dtype), logits_dtype)
    logits = logits.reshape(T, E)
    ids, sel = topk_select(logits, k)
    gates = gates_from_selected(sel).to(compute_dtype)
    ids_flat = ids.reshape(-1)
    counts, starts = counts_offsets(ids_flat, E)
    pos_to_row, row_to_pos = stable_permutation(ids_flat)
    xp = x2[torch.from_numpy(pos_to_row // k)]
    ffn = expert_ffn_rows(xp, starts, w1.to(compute_dtype), w3.to(compute_dtype),
                          w2.to(compute_dtype), emulate_bf16)
    out = combine_rows(ffn["y"], gates.reshape(-1), row_to_pos, T, k)
    res = {"logits": logits, "ids": ids, "sel_logits": sel, "gates": gates, "counts": counts,
           "starts": starts, "pos_to_row": pos_to_row, "row_to_pos": row_to_pos, "xp": xp,
           "out": out.reshape(shape), "x2": x2, "k": k}
    res.update(ffn)
    return res


def moe_backward(fwd: dict, dy: torch.Tensor, wr: torch.Tensor, w1: torch.Tensor,
                 w3: torch.Tensor, w2: torch.Tensor, emulate_bf16: bool = False) -> dict:
    """Hand-derived backward of `moe_forward` (the reference has no source for it: it is
    autograd through mlp.py:95-169).  Every intermediate gradient is returned by name.

    pinned by: torch.autograd through `moe_forward_autograd` (library), fp64 gradcheck on
    tiny shapes, central finite differences; invariants (zero grad slices for empty
    experts, sum_j dsel[t,j] == 0).
    """
    cd = fwd["x2"].dtype
    x2, k = fwd["x2"], fwd["k"]
    T, H = x2.shape
    E = wr.shape[0]
    dy2 = dy.reshape(T, H).to(cd)
    gates = fwd["gates"]
    pos_to_row = torch.from_numpy(fwd["pos_to_row"])
    row_to_pos = torch.from_numpy(fwd["row_to_pos"])
    tok_of_pos = pos_to_row // k
    starts = fwd["starts"]
    w1c, w3c, w2c, wrc = (w.to(cd) for w in (w1, w3, w2, wr))

    # combine backward (mlp.py:166-167): rows*gate summed over k
    gate_of_pos = gates.reshape(-1)[pos_to_row]
    dyp = _maybe_round(dy2[tok_of_pos] * gate_of_pos.unsqueeze(-1), emulate_bf16)
    dgate_pos = (dy2[tok_of_pos] * fwd["y"]).sum(-1)

    g, u, act, xp = fwd["g"], fwd["u"], fwd["act"], fwd["xp"]
    dg = torch.zeros_like(g)
    du = torch.zeros_like(u)
    dxp = torch.zeros_like(xp)
    dw1 = torch.zeros_like(w1c)
    dw3 = torch.zeros_like(w3c)
    dw2 = torch.zeros_like(w2c)
    for e in range(E):
        a, b = int(starts[e]), int(starts[e + 1])
        if a == b:
            continue
        dact = dyp[a:b] @ w2c[e]                      # [n,H]@[H,I]
        dw2[e] = dyp[a:b].t() @ act[a:b]              # [H,n]@[n,I]
        sig = torch.sigmoid(g[a:b])
        silu = g[a:b] * sig
        if emulate_bf16:
            # the device takes the gate gradient from here: dyp carries the gate (and its bf16
            # rounding), so <dact, act> = gate * <dy, y>; y itself is not read again
            gp = gate_of_pos[a:b]
            raw = (dact * (silu * u[a:b])).sum(-1)
            dgate_pos[a:b] = torch.where(gp != 0, raw / gp, torch.zeros_like(raw))
        dge = _maybe_round(dact * u[a:b] * (sig * (1 + g[a:b] * (1 - sig))), emulate_bf16)
        due = _maybe_round(dact * silu, emulate_bf16)
        dg[a:b], du[a:b] = dge, due
        dxp[a:b] = _maybe_round(dge @ w1c[e] + due @ w3c[e], emulate_bf16)
        dw1[e] = dge.t() @ xp[a:b]
        dw3[e] = due.t() @ xp[a:b]
    dgates = dgate_pos[row_to_pos].reshape(T, k)
    # repeat_interleave backward (mlp.py:104): sum the k row-grads of a token, slot order
    dx_expert = dxp[row_to_pos].view(T, k, H).sum(1)
    # softmax-over-k backward, then topk backward scatters into zeros (mlp.py:101-102)
    dsel = gates * (dgates - (gates * dgates).sum(-1, keepdim=True))
    dlogits = torch.zeros(T, E, dtype=cd)
    dlogits.scatter_(1, torch.from_numpy(fwd["ids"]), dsel)
    dlogits_used = dlogits
    if emulate_bf16:
        dlogits_used = _maybe_round(dlogits, True)
    dwr = dlogits_used.t() @ x2
    # (the router path's input gradient is a bf16 library product on the device)
    dx_router = _maybe_round(dlogits_used @ wrc, emulate_bf16)
    return {"dyp": dyp, "dgates": dgates, "dg": dg, "du": du, "dxp": dxp, "dw1": dw1,
            "dw3": dw3, "dw2": dw2, "dx_expert": dx_expert, "dsel": dsel, "dlogits": dlogits,
            "dwr": dwr, "dx_router": dx_router, "dx": (dx_expert + dx_router).reshape(dy.shape),
            "dbias": dlogits_used.sum(0)}


def moe_forward_autograd(x, wr, w1, w3, w2, k, ids: np.ndarray | None = None):
    """Differentiable torch restatement used only to pin `moe_backward` through the
    library's autograd: same math as `moe_forward`, routing ids frozen (they are
    piecewise constant), everything else built from differentiable torch ops."""
    T, H = x.shape
    E = wr.shape[0]
    logits = F.linear(x, wr)
    if ids is None:
        ids, _ = topk_select(logits, k)
    ids_t = torch.from_numpy(ids)
    gates = F.softmax(torch.gather(logits, 1, ids_t), dim=-1)
    ids_flat = ids.reshape(-1)
    _, starts = counts_offsets(ids_flat, E)
    pos_to_row, row_to_pos = stable_permutation(ids_flat)
    xp = x[torch.from_numpy(pos_to_row // k)]
    ys = []
    for e in range(E):
        a, b = int(starts[e]), int(starts[e + 1])
        xe = xp[a:b]
        ys.append(F.linear(F.silu(F.linear(xe, w1[e])) * F.linear(xe, w3[e]), w2[e]))
    y = torch.cat(ys, 0)
    rows = y[torch.from_numpy(row_to_pos)] * gates.reshape(-1, 1)
    return rows.view(T, k, H).sum(1)


def moe_forward_padded_bmm(x, wr, w1, w3, w2, k, logits: torch.Tensor | None = None):
    """Literal restatement of the live branch of the reference, mlp.py:100-167 with the
    zero-padded `bmm`s of mlp.py:133-158, on one rank (the all-to-alls of :113-120,:162 are
    identity copies; the EP-rank sort of :106-109 has a single key).  fp32, no autocast.
    Exists to show the per-expert loop oracle and the reference's formulation agree
    (padding rows contribute exactly zero)."""
    T, D = x.shape
    E = wr.shape[0]
    if logits is None:
        logits = F.linear(x, wr)
    ids, sel = topk_select(logits, k)
    weights = F.softmax(sel.float(), dim=-1).view(-1).to(x.dtype)
    selected = torch.from_numpy(ids).view(-1)
    flat_x = x.repeat_interleave(k, dim=0)
    sort_idx = torch.argsort(selected, stable=True)
    local_x = flat_x[sort_idx]
    local_e = selected[sort_idx]
    counts = torch.bincount(local_e, minlength=E)
    offs = torch.cumsum(counts, 0).to(torch.int32)
    max_tokens = int(counts.max())
    starts = torch.zeros_like(offs)
    starts[1:] = offs[:-1]
    rel = torch.arange(len(local_x)) - starts[local_e]
    padded = torch.zeros(E, max_tokens, D, dtype=x.dtype).index_put((local_e, rel), local_x)
    gate_out = torch.bmm(padded, w1.transpose(1, 2))
    up_out = torch.bmm(padded, w3.transpose(1, 2))
    act = F.silu(gate_out) * up_out
    down = torch.bmm(act, w2.transpose(1, 2))[local_e, rel]
    unperm = down[torch.argsort(sort_idx)] * weights.unsqueeze(-1)
    return unperm.view(T, k, D).sum(1)


def experts_rows_forward(rows: torch.Tensor, ids: np.ndarray, w1, w3, w2,
                         compute_dtype=torch.float32, emulate_bf16: bool = False) -> dict:
    """Post-dispatch entry: the state at mlp.py:122 (`received_x`, `received_experts` as
    local ids) to the state at mlp.py:161 (`out_x`, rows back in arrival order)."""
    E = w1.shape[0]
    counts, starts = counts_offsets(ids, E)
    pos_to_row, row_to_pos = stable_permutation(ids)
    xp = rows.to(compute_dtype)[torch.from_numpy(pos_to_row)]
    ffn = expert_ffn_rows(xp, starts, w1.to(compute_dtype), w3.to(compute_dtype),
                          w2.to(compute_dtype), emulate_bf16)
    out = ffn["y"][torch.from_numpy(row_to_pos)]
    res = {"counts": counts, "starts": starts, "pos_to_row": pos_to_row,
           "row_to_pos": row_to_pos, "xp": xp, "out": out}
    res.update(ffn)
    return res


def experts_rows_backward(fwd: dict, dout: torch.Tensor, w1, w3, w2,
                          emulate_bf16: bool = False) -> dict:
    """Backward of `experts_rows_forward` w.r.t. the rows and the three weight stacks."""
    cd = fwd["xp"].dtype
    starts = fwd["starts"]
    pos_to_row = torch.from_numpy(fwd["pos_to_row"])
    row_to_pos = torch.from_numpy(fwd["row_to_pos"])
    dyp = _maybe_round(dout.to(cd)[pos_to_row], emulate_bf16)
    w1c, w3c, w2c = (w.to(cd) for w in (w1, w3, w2))
    g, u, act, xp = fwd["g"], fwd["u"], fwd["act"], fwd["xp"]
    dxp = torch.zeros_like(xp)
    dw1, dw3, dw2 = torch.zeros_like(w1c), torch.zeros_like(w3c), torch.zeros_like(w2c)
    for e in range(w1c.shape[0]):
        a, b = int(starts[e]), int(starts[e + 1])
        if a == b:
            continue
        dact = dyp[a:b] @ w2c[e]
        dw2[e] = dyp[a:b].t() @ act[a:b]
        sig = torch.sigmoid(g[a:b])
        dge = _maybe_round(dact * u[a:b] * (sig * (1 + g[a:b] * (1 - sig))), emulate_bf16)
        due = _maybe_round(dact * (g[a:b] * sig), emulate_bf16)
        dxp[a:b] = _maybe_round(dge @ w1c[e] + due @ w3c[e], emulate_bf16)
        dw1[e] = dge.t() @ xp[a:b]
        dw3[e] = due.t() @ xp[a:b]
    return {"drows": dxp[row_to_pos], "dw1": dw1, "dw3": dw3, "dw2": dw2}
