"""Pins for every function of oracle/moe_oracle.py (CPU only).

The reference ships no tests or golden vectors, so each pin is a closed form, an
invariant, a brute force on tiny inputs or an independent library routine, chosen so that
a plausible slip (dropped term, wrong sign or index, transposed operand) fails one.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


def _mk(T, H, E, I, seed=0, dtype=torch.float32, std=0.3):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, H, generator=g, dtype=dtype)
    wr = torch.randn(E, H, generator=g, dtype=dtype) * std
    w1 = torch.randn(E, I, H, generator=g, dtype=dtype) * std
    w3 = torch.randn(E, I, H, generator=g, dtype=dtype) * std
    w2 = torch.randn(E, H, I, generator=g, dtype=dtype) * std
    return x, wr, w1, w3, w2


# ----------------------------------------------------------------------------- top-k
def _topk_bruteforce(row, k):
    """Selection by repeated scan: best = larger logit, then smaller index."""
    chosen = []
    for _ in range(k):
        best = None
        for e, v in enumerate(row):
            if e in chosen:
                continue
            if best is None or v > row[best]:
                best = e
        chosen.append(best)
    return chosen


def test_topk_bruteforce_with_ties():
    rng = np.random.default_rng(1)
    for _ in range(200):
        E = int(rng.integers(2, 12))
        k = int(rng.integers(1, E + 1))
        row = rng.integers(-3, 3, size=E).astype(np.float32)  # many exact ties
        ids, sel = O.topk_select(torch.from_numpy(row)[None], k)
        assert ids[0].tolist() == _topk_bruteforce(row.tolist(), k)
        assert sel[0].tolist() == [row[i] for i in ids[0]]


def test_topk_documented_tie_example():
    # lower expert index wins among equal logits; slots stay in descending-logit order
    ids, _ = O.topk_select(torch.tensor([[1.0, 2.0, 2.0, 0.5, 2.0, 1.0]]), 2)
    assert ids.tolist() == [[1, 2]]
    ids, _ = O.topk_select(torch.tensor([[1.0, 2.0, 2.0, 0.5, 2.0, 1.0]]), 5)
    assert ids.tolist() == [[1, 2, 4, 0, 5]]


def test_topk_matches_torch_on_tie_free_rows():
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(512, 64, generator=g).to(torch.bfloat16)
    k = 8
    ids, sel = O.topk_select(logits, k)
    tv, ti = torch.topk(logits, k, dim=-1)
    srt = torch.sort(logits.float(), dim=-1, descending=True).values[:, :k + 1]
    tie_free = (srt[:, 1:] != srt[:, :-1]).all(-1)
    assert tie_free.sum() > 50 and (~tie_free).sum() > 5  # both kinds present
    assert np.array_equal(ids[tie_free.numpy()], ti[tie_free].numpy())
    assert torch.equal(sel.float(), tv.float())  # value multiset (sorted) equal on all rows
    assert all(len(set(r)) == k for r in ids.tolist())


def test_topk_non_finite_matches_torch():
    """NaN ranks above every number and -inf below (torch.topk's order, mlp.py:101), whatever the
    NaN's sign bit; checked against the library routine on fp32 rows without ties."""
    g = torch.Generator().manual_seed(31)
    logits = torch.randn(64, 32, generator=g)
    inf = float("inf")
    logits[0, 3] = float("nan")
    logits[1, 7] = torch.tensor([0xffc00000 - (1 << 32)], dtype=torch.int32).view(torch.float32).item()  # sign set
    logits[2, 5] = inf
    logits[3, 10:] = -inf            # 10 finite logits, k = 8: still no tie among the selected
    logits[4, 0] = float("nan")
    logits[4, 1] = inf
    k = 8
    ids, sel = O.topk_select(logits, k)
    tv, ti = torch.topk(logits, k, dim=-1)
    assert np.array_equal(ids, ti.numpy())
    assert torch.equal(torch.nan_to_num(sel, nan=123.0), torch.nan_to_num(tv, nan=123.0))
    assert ids[0, 0] == 3 and ids[1, 0] == 7 and ids[4, :2].tolist() == [0, 1]
    gates = O.gates_from_selected(sel)
    assert torch.isnan(gates[[0, 1, 2, 4]]).all() and torch.isfinite(gates[3]).all()


def test_gates_invariants():
    g = torch.Generator().manual_seed(4)
    logits = torch.randn(64, 16, generator=g)
    ids, sel = O.topk_select(logits, 4)
    gates = O.gates_from_selected(sel)
    assert torch.allclose(gates.sum(-1), torch.ones(64), atol=1e-6)
    # softmax over all experts -> top-k -> renormalise  ==  top-k -> softmax
    p = F.softmax(logits, -1)
    pk = torch.gather(p, 1, torch.from_numpy(ids))
    assert torch.allclose(pk / pk.sum(-1, keepdim=True), gates, atol=1e-6)
    assert torch.equal(O.gates_from_selected(sel[:, :1]), torch.ones(64, 1))
    eq = O.gates_from_selected(torch.tensor([[2.0, 2.0, 1.0]]))
    assert eq[0, 0] == eq[0, 1] > eq[0, 2]


# ----------------------------------------------------------------------------- dispatch
def test_counts_offsets_and_permutation_bruteforce():
    rng = np.random.default_rng(5)
    for _ in range(50):
        E = int(rng.integers(1, 9))
        R = int(rng.integers(0, 40))
        ids = rng.integers(0, E, size=R)
        counts, starts = O.counts_offsets(ids, E)
        assert counts.tolist() == [int((ids == e).sum()) for e in range(E)]
        assert starts[0] == 0 and starts[-1] == R and (np.diff(starts) == counts).all()
        p2r, r2p = O.stable_permutation(ids)
        brute = [r for e in range(E) for r in range(R) if ids[r] == e]  # counting sort
        assert p2r.tolist() == brute
        assert (p2r[r2p] == np.arange(R)).all() and (r2p[p2r] == np.arange(R)).all()
        assert (np.diff(ids[p2r]) >= 0).all()


def test_permutation_equals_composed_reference_sorts():
    # mlp.py:107 (sort by EP rank, one rank -> single key) then :123 (sort by local id)
    rng = np.random.default_rng(6)
    ids = torch.from_numpy(rng.integers(0, 8, size=300))
    g_idx = torch.argsort(ids // 8, stable=True)
    l_idx = torch.argsort((ids[g_idx] % 8), stable=True)
    p2r, r2p = O.stable_permutation(ids.numpy())
    assert torch.equal(g_idx[l_idx], torch.from_numpy(p2r))
    # inverse == argsort(local_sort_idx) composed with argsort(global_sort_idx) (:160,:163)
    inv = torch.argsort(l_idx)[torch.argsort(g_idx)]
    assert torch.equal(inv, torch.from_numpy(r2p))


# ----------------------------------------------------------------------------- experts
def test_single_expert_is_dense_mlp():
    x, wr, w1, w3, w2 = _mk(20, 16, 1, 12, seed=7)
    out = O.moe_forward(x, wr, w1, w3, w2, k=1)["out"]
    dense = F.linear(F.silu(F.linear(x, w1[0])) * F.linear(x, w3[0]), w2[0])  # mlp.py:44
    assert torch.allclose(out, dense, atol=1e-6)


def test_identical_experts_reduce_to_dense_mlp_for_any_routing():
    x, wr, w1, w3, w2 = _mk(33, 16, 5, 12, seed=8)
    w1 = w1[:1].expand(5, -1, -1).contiguous()
    w3 = w3[:1].expand(5, -1, -1).contiguous()
    w2 = w2[:1].expand(5, -1, -1).contiguous()
    out = O.moe_forward(x, wr, w1, w3, w2, k=3)["out"]  # gates sum to 1
    dense = F.linear(F.silu(F.linear(x, w1[0])) * F.linear(x, w3[0]), w2[0])
    assert torch.allclose(out, dense, atol=1e-5)


def test_loop_oracle_equals_padded_bmm_restatement():
    for seed, (T, H, E, I, k) in enumerate([(16, 32, 4, 24, 2), (40, 16, 6, 8, 3), (9, 8, 8, 8, 1)]):
        x, wr, w1, w3, w2 = _mk(T, H, E, I, seed=20 + seed)
        a = O.moe_forward(x, wr, w1, w3, w2, k)["out"]
        b = O.moe_forward_padded_bmm(x, wr, w1, w3, w2, k)
        assert torch.allclose(a, b, atol=1e-5, rtol=1e-5)


def test_empty_experts_contribute_nothing_and_get_zero_grads():
    x, wr, w1, w3, w2 = _mk(12, 8, 6, 8, seed=9)
    logits = torch.full((12, 6), -5.0)
    logits[:, 1] = 1.0
    logits[:, 4] = 2.0  # only experts 4 and 1 ever selected
    f = O.moe_forward(x, wr, w1, w3, w2, k=2, logits=logits)
    assert f["counts"].tolist() == [0, 12, 0, 0, 12, 0]
    assert (f["ids"] == np.array([4, 1])).all()
    b = O.moe_backward(f, torch.ones_like(x), wr, w1, w3, w2)
    for e in (0, 2, 3, 5):
        assert not b["dw1"][e].any() and not b["dw3"][e].any() and not b["dw2"][e].any()
    assert b["dw1"][1].abs().sum() > 0


def test_grouped_mm_library_crosscheck():
    if not hasattr(F, "grouped_mm"):
        pytest.skip("torch has no grouped_mm")
    x, wr, w1, w3, w2 = _mk(64, 32, 4, 16, seed=10)
    f = O.moe_forward(x, wr, w1, w3, w2, k=2)
    offs = torch.from_numpy(f["starts"][1:].copy())
    xb = f["xp"].to(torch.bfloat16)
    try:
        g = F.grouped_mm(xb, w1.to(torch.bfloat16).transpose(1, 2), offs=offs)
    except Exception as e:  # library routine unavailable on this build
        pytest.skip(f"grouped_mm not runnable on CPU here: {e}")
    assert torch.allclose(g.float(), f["g"], atol=5e-2, rtol=5e-2)


# ----------------------------------------------------------------------------- combine
def test_combine_k1_is_pure_unpermute_and_linear():
    rng = np.random.default_rng(11)
    ids = rng.integers(0, 4, size=10)
    p2r, r2p = O.stable_permutation(ids)
    y = torch.arange(10.0).unsqueeze(-1).repeat(1, 3)
    out = O.combine_rows(y, torch.ones(10), r2p, 10, 1)
    assert torch.equal(out[:, 0], torch.from_numpy(r2p).float())
    T, k = 5, 2
    y = torch.randn(10, 3)
    gts = torch.rand(10)
    out = O.combine_rows(y, gts, r2p, T, k)
    for t in range(T):
        exp = sum(gts[t * k + j] * y[r2p[t * k + j]] for j in range(k))
        assert torch.allclose(out[t], exp, atol=1e-6)


# ----------------------------------------------------------------------------- backward
@pytest.mark.parametrize("T,H,E,I,k", [(16, 32, 4, 24, 2), (24, 16, 8, 8, 3), (8, 8, 3, 8, 1)])
def test_manual_backward_matches_autograd(T, H, E, I, k):
    x, wr, w1, w3, w2 = (t.double() for t in _mk(T, H, E, I, seed=30 + T))
    dy = torch.randn(T, H, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    f = O.moe_forward(x, wr, w1, w3, w2, k, compute_dtype=torch.float64)
    b = O.moe_backward(f, dy, wr, w1, w3, w2)
    leaves = [t.clone().requires_grad_(True) for t in (x, wr, w1, w3, w2)]
    out = O.moe_forward_autograd(*leaves, k, ids=f["ids"])
    assert torch.allclose(out, f["out"], atol=1e-10)
    out.backward(dy)
    for name, leaf in zip(("dx", "dwr", "dw1", "dw3", "dw2"), leaves):
        assert torch.allclose(b[name], leaf.grad, atol=1e-9, rtol=1e-9), name
    # softmax Jacobian: selected-logit grads of a token sum to zero
    assert torch.allclose(b["dsel"].sum(-1), torch.zeros(T, dtype=torch.float64), atol=1e-10)
    # dx = expert term + router term: with the gates frozen only the expert term remains
    leaves = [t.clone().requires_grad_(True) for t in (x, w1, w3, w2)]
    ids_flat = f["ids"].reshape(-1)
    xp = leaves[0][torch.from_numpy(f["pos_to_row"] // k)]
    ys = []
    for e in range(E):
        a, bb = int(f["starts"][e]), int(f["starts"][e + 1])
        ys.append(F.linear(F.silu(F.linear(xp[a:bb], leaves[1][e])) * F.linear(xp[a:bb], leaves[2][e]), leaves[3][e]))
    rows = torch.cat(ys)[torch.from_numpy(f["row_to_pos"])] * f["gates"].reshape(-1, 1)
    rows.view(T, k, H).sum(1).backward(dy)
    assert torch.allclose(b["dx_expert"], leaves[0].grad, atol=1e-9)


def test_bias_gradient_is_the_column_sum_of_dlogits_by_finite_differences():
    """`moe_backward()["dbias"]`: the per-expert router bias enters as logit + bias, so its
    gradient must equal d<dy, out>/d bias, taken here by central differences in fp64 (routing
    frozen by the margin between the k-th and (k+1)-th logit being far above the step)."""
    T, H, E, I, k = 12, 16, 6, 8, 2
    x, wr, w1, w3, w2 = (t.double() for t in _mk(T, H, E, I, seed=77))
    bias = torch.randn(E, dtype=torch.float64, generator=torch.Generator().manual_seed(3)) * 0.5
    dy = torch.randn(T, H, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    f = O.moe_forward(x, wr, w1, w3, w2, k, bias=bias, compute_dtype=torch.float64)
    b = O.moe_backward(f, dy, wr, w1, w3, w2)
    srt = torch.sort(F.linear(x, wr) + bias, dim=-1, descending=True).values
    assert (srt[:, k - 1] - srt[:, k]).min() > 1e-3
    h = 1e-6
    for e in range(E):
        d = torch.zeros(E, dtype=torch.float64)
        d[e] = h
        fp = O.moe_forward(x, wr, w1, w3, w2, k, bias=bias + d, compute_dtype=torch.float64)
        fm = O.moe_forward(x, wr, w1, w3, w2, k, bias=bias - d, compute_dtype=torch.float64)
        assert np.array_equal(fp["ids"], f["ids"]) and np.array_equal(fm["ids"], f["ids"])
        fd = ((fp["out"] - fm["out"]) * dy).sum().item() / (2 * h)
        assert abs(fd - b["dbias"][e].item()) <= 1e-6 * max(1.0, abs(fd)), (e, fd, b["dbias"][e].item())
    # and it is not trivially zero, nor is any bias without effect
    assert b["dbias"].abs().min() > 1e-4
    assert abs(b["dbias"].sum().item()) < 1e-9   # the softmax over the selected logits is shift-invariant


def test_gradcheck_fp64_tiny():
    T, H, E, I, k = 6, 8, 4, 8, 2
    x, wr, w1, w3, w2 = (t.double() for t in _mk(T, H, E, I, seed=40, std=0.5))
    ids, _ = O.topk_select(F.linear(x, wr), k)
    srt = torch.sort(F.linear(x, wr), -1, descending=True).values
    assert (srt[:, k - 1] - srt[:, k]).min() > 1e-3  # away from routing ties
    leaves = [t.clone().requires_grad_(True) for t in (x, wr, w1, w3, w2)]
    assert torch.autograd.gradcheck(lambda *a: O.moe_forward_autograd(*a, k, ids=ids), leaves,
                                    eps=1e-6, atol=1e-5)


def test_finite_difference_on_weight_slices():
    T, H, E, I, k = 10, 8, 3, 8, 2
    x, wr, w1, w3, w2 = (t.double() for t in _mk(T, H, E, I, seed=41, std=0.5))
    dy = torch.randn(T, H, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    f = O.moe_forward(x, wr, w1, w3, w2, k, compute_dtype=torch.float64)
    b = O.moe_backward(f, dy, wr, w1, w3, w2)
    logits = f["logits"]

    def loss(w1_, w3_, w2_):
        return (O.moe_forward(x, wr, w1_, w3_, w2_, k, logits=logits,
                              compute_dtype=torch.float64)["out"] * dy).sum()
    eps = 1e-6
    for name, idx in (("dw1", (1, 2, 3)), ("dw3", (0, 5, 1)), ("dw2", (2, 4, 6))):
        ws = [w1.clone(), w3.clone(), w2.clone()]
        j = ("dw1", "dw3", "dw2").index(name)
        ws[j][idx] += eps
        up = loss(*ws)
        ws[j][idx] -= 2 * eps
        dn = loss(*ws)
        assert abs((up - dn) / (2 * eps) - b[name][idx]) < 1e-6, name


def test_rows_entry_forward_backward():
    rng = np.random.default_rng(12)
    E, H, I, R = 5, 16, 8, 50
    _, _, w1, w3, w2 = (t.double() for t in _mk(1, H, E, I, seed=42))
    rows = torch.randn(R, H, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    ids = rng.integers(0, E, size=R)
    ids[ids == 2] = 3  # expert 2 empty
    dout = torch.randn(R, H, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    f = O.experts_rows_forward(rows, ids, w1, w3, w2, compute_dtype=torch.float64)
    b = O.experts_rows_backward(f, dout, w1, w3, w2)
    leaves = [t.clone().requires_grad_(True) for t in (rows, w1, w3, w2)]
    out = torch.stack([F.linear(F.silu(F.linear(leaves[0][r], leaves[1][ids[r]])) *
                                F.linear(leaves[0][r], leaves[2][ids[r]]), leaves[3][ids[r]])
                       for r in range(R)])  # row-by-row, no permutation at all
    assert torch.allclose(out, f["out"], atol=1e-10)
    out.backward(dout)
    for name, leaf in zip(("drows", "dw1", "dw3", "dw2"), leaves):
        assert torch.allclose(b[name], leaf.grad, atol=1e-9), name
    assert not b["dw1"][2].any()


# ----------------------------------------------------------------------------- bf16 storage emulation
def _rb(t):
    return t.to(torch.bfloat16).to(t.dtype)


class _RoundValue(torch.autograd.Function):
    """bf16 rounding of the value; the gradient passes unchanged."""
    @staticmethod
    def forward(ctx, t):
        return _rb(t)

    @staticmethod
    def backward(ctx, gr):
        return gr


class _RoundGrad(torch.autograd.Function):
    """The value passes unchanged; the gradient is rounded to bf16."""
    @staticmethod
    def forward(ctx, t):
        return t.view_as(t)

    @staticmethod
    def backward(ctx, gr):
        return _rb(gr)


class _StoredSwiGLU(torch.autograd.Function):
    """act = bf16(silu(g) * u) from unrounded g, u; backward differentiates silu(g)*u with the
    library's autograd AT the bf16-stored g, u and rounds both results to bf16."""
    @staticmethod
    def forward(ctx, g, u):
        ctx.save_for_backward(_rb(g), _rb(u))
        return _rb(F.silu(g) * u)

    @staticmethod
    def backward(ctx, dact):
        gs, us = (t.detach().requires_grad_(True) for t in ctx.saved_tensors)
        with torch.enable_grad():
            a = F.silu(gs) * us
        dg, du = torch.autograd.grad(a, (gs, us), dact)
        return _rb(dg), _rb(du)


@pytest.mark.parametrize("T,H,E,I,k", [(96, 64, 6, 48, 2), (40, 32, 4, 24, 3), (64, 48, 5, 40, 1)])
def test_bf16_emulation_matches_an_autograd_restatement_with_the_same_rounding_points(T, H, E, I, k):
    """The oracle's `emulate_bf16` mode (the yardstick of the GPU tolerance rule) against an
    independent restatement: the reference's padded-bmm formulation (mlp.py:133-167) under the
    library's autograd, with bf16 rounding inserted as autograd nodes at the points where the
    device stores bf16 (g, u, act, y forward; gate*dy, dg, du, d rows, dlogits backward).  Values
    that do not depend on how the gate gradient is formed must agree to fp32 summation order; the
    gate gradient itself is <dy, y> here and <dact, act>/gate there (equal in exact arithmetic),
    so it and what follows from it agree to bf16 rounding."""
    x, wr, w1, w3, w2 = (_rb(t) for t in _mk(T, H, E, I, seed=70 + T, std=0.2))
    dy = _rb(torch.randn(T, H, generator=torch.Generator().manual_seed(5)))
    logits = _rb(F.linear(x, wr))
    fe = O.moe_forward(x, wr, w1, w3, w2, k, logits=logits, emulate_bf16=True)
    be = O.moe_backward(fe, dy, wr, w1, w3, w2, emulate_bf16=True)

    ids = torch.from_numpy(fe["ids"])
    lx, lw1, lw3, lw2 = (t.clone().requires_grad_(True) for t in (x, w1, w3, w2))
    llog = logits.clone().requires_grad_(True)
    weights = F.softmax(torch.gather(llog, 1, ids).float(), dim=-1).view(-1)
    selected = ids.view(-1)
    flat_x = lx.repeat_interleave(k, dim=0)
    sort_idx = torch.argsort(selected, stable=True)
    local_x = _RoundGrad.apply(flat_x[sort_idx])
    local_e = selected[sort_idx]
    counts = torch.bincount(local_e, minlength=E)
    starts = torch.cumsum(counts, 0) - counts
    rel = torch.arange(T * k) - starts[local_e]
    padded = torch.zeros(E, int(counts.max()), H).index_put((local_e, rel), local_x)
    act = _StoredSwiGLU.apply(torch.bmm(padded, lw1.transpose(1, 2)), torch.bmm(padded, lw3.transpose(1, 2)))
    down = _RoundGrad.apply(_RoundValue.apply(torch.bmm(act, lw2.transpose(1, 2))[local_e, rel]))
    out = (down[torch.argsort(sort_idx)] * weights.unsqueeze(-1)).view(T, k, H).sum(1)
    assert torch.allclose(out, fe["out"], rtol=1e-5, atol=1e-6)
    out.backward(dy)

    tight = dict(rtol=2e-5, atol=2e-6)
    assert torch.allclose(lw1.grad, be["dw1"], **tight)
    assert torch.allclose(lw3.grad, be["dw3"], **tight)
    assert torch.allclose(lw2.grad, be["dw2"], **tight)
    assert torch.allclose(lx.grad, be["dx_expert"], **tight)   # router path not in this graph's x
    # gate-gradient side: two estimators of the same number, a bf16 rounding apart
    dl = llog.grad
    scale = be["dlogits"].abs().max().item()
    assert (dl - be["dlogits"]).abs().max().item() <= 2e-2 * scale
    dl_r = _rb(dl)
    assert ((dl_r.t() @ x) - be["dwr"]).norm() <= 2e-2 * be["dwr"].norm()
    assert ((dl_r @ wr) - be["dx_router"]).norm() <= 2e-2 * be["dx_router"].norm()
    # and the emulation differs from the unrounded oracle (it is not a no-op) by bf16-sized amounts
    f = O.moe_forward(x, wr, w1, w3, w2, k, logits=logits)
    b = O.moe_backward(f, dy, wr, w1, w3, w2)
    for n in ("dw1", "dw3", "dw2"):
        rel_err = ((be[n] - b[n]).norm() / b[n].norm()).item()
        assert 1e-5 < rel_err < 1e-2, (n, rel_err)


def test_bf16_emulation_of_the_rows_entry_matches_the_layer_emulation():
    """`experts_rows_*` with `emulate_bf16` is the k = 1, gate = 1 case of the layer's emulation
    (pinned above): same dyp, dg, du, d rows and weight gradients."""
    T, H, E, I = 80, 32, 5, 24
    x, wr, w1, w3, w2 = (_rb(t) for t in _mk(T, H, E, I, seed=90, std=0.2))
    dy = _rb(torch.randn(T, H, generator=torch.Generator().manual_seed(6)))
    logits = _rb(F.linear(x, wr))
    fe = O.moe_forward(x, wr, w1, w3, w2, 1, logits=logits, emulate_bf16=True)
    be = O.moe_backward(fe, dy, wr, w1, w3, w2, emulate_bf16=True)
    assert torch.equal(fe["gates"], torch.ones(T, 1))
    ids = fe["ids"].reshape(-1)
    fr = O.experts_rows_forward(x, ids, w1, w3, w2, emulate_bf16=True)
    br = O.experts_rows_backward(fr, dy, w1, w3, w2, emulate_bf16=True)
    assert torch.equal(fr["out"], fe["out"])
    assert torch.equal(br["drows"], be["dx_expert"])
    for n in ("dw1", "dw3", "dw2"):
        assert torch.equal(br[n], be[n]), n


def test_oracle_reproduces_its_committed_fixture():
    """tests/golden/oracle_tiny.npz holds what the oracle computed (both modes, forward and
    backward) on seeded tiny inputs when the fixture was made: an edit that changes what the
    oracle computes fails here until the fixture is regenerated on purpose."""
    import importlib.util
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_oracle_fixture", os.path.join(here, "make_oracle_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    want = np.load(os.path.join(here, "oracle_tiny.npz"))
    got = mod.compute()
    assert set(want.files) == set(got)
    for k in want.files:
        if want[k].dtype.kind in "iu":
            assert np.array_equal(want[k], got[k]), k
        else:
            assert np.allclose(want[k], got[k], rtol=1e-5, atol=1e-6), k


# ----------------------------------------------------------------------------- block oracle
def test_block_oracle_pieces():
    from oracle import block_oracle as B
    g = torch.Generator().manual_seed(50)
    x = torch.randn(2, 12, 32, generator=g)
    w = torch.rand(32, generator=g) + 0.5
    ref = w * x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6)
    assert torch.allclose(B.rmsnorm(x, w), ref, atol=1e-6)
    # RoPE: position 0 untouched; each (d, d + hd/2) pair is rotated, so its norm is kept
    # only where the duplicated cos/sin layout happens to pair equal angles; what always
    # holds is linearity and the identity at position 0
    q = torch.randn(1, 2, 5, 8, generator=g)
    k = torch.randn(1, 2, 5, 8, generator=g)
    q2, k2 = B.rope(q, k)
    assert torch.allclose(q2[..., 0, :], q[..., 0, :]) and torch.allclose(k2[..., 0, :], k[..., 0, :])
    qa, _ = B.rope(2 * q, k)
    assert torch.allclose(qa, 2 * q2, atol=1e-6)
    # element by element, as attn.py:53-54 and :61-63 write it for head_dim 4 at position p:
    # cos = [c0, c0, c1, c1] (interleave-duplicated), rotate_half(q) = [-q2, -q3, q0, q1]
    # (split in halves), so out = [q0 c0 - q2 s0, q1 c0 - q3 s0, q2 c1 + q0 s1, q3 c1 + q1 s1]
    # with angle_i = p * theta^(-2i/4).  A layout that pairs (0,1),(2,3) or duplicates the angles
    # as [c0, c1, c0, c1] gives different numbers.
    import math
    q4 = torch.tensor([[[[0.0, 0.0, 0.0, 0.0], [0.0, 0.0, 0.0, 0.0], [0.0, 0.0, 0.0, 0.0], [1.0, 2.0, 3.0, 4.0]]]])
    r4, _ = B.rope(q4, q4)
    a0, a1 = 3.0, 3.0 * 10000.0 ** (-0.5)
    want = [1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a0) - 4 * math.sin(a0),
            3 * math.cos(a1) + 1 * math.sin(a1), 4 * math.cos(a1) + 2 * math.sin(a1)]
    assert torch.allclose(r4[0, 0, 3], torch.tensor(want), atol=1e-5)
    # attention against the library's fused routine on the CPU
    nh, nkv, C = 4, 2, 32
    ws = [torch.randn(o, C, generator=g) * 0.2 for o in (C, C // 2, C // 2, C)]
    y = B.attention(x, *ws, nh, nkv)
    hd = C // nh
    qq = F.linear(x, ws[0]).view(2, 12, nh, hd).transpose(1, 2)
    kk = F.linear(x, ws[1]).view(2, 12, nkv, hd).transpose(1, 2).repeat_interleave(2, 1)
    vv = F.linear(x, ws[2]).view(2, 12, nkv, hd).transpose(1, 2).repeat_interleave(2, 1)
    qq, kk = B.rope(qq, kk)
    lib = F.scaled_dot_product_attention(qq, kk, vv, is_causal=True)
    assert torch.allclose(y, F.linear(lib.transpose(1, 2).reshape(2, 12, C), ws[3]), atol=1e-5)
