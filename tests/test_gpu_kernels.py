"""GPU parity tests, one group per exported kernel family, called through the C ABI
(ops.py is a thin ctypes wrapper) and checked against oracle/moe_oracle.py.

Bars: integer outputs (ids, counts, offsets, permutation, pure row copies) bit-exact;
floating point within rtol = atol = 1e-2 of the fp32 oracle on identical bf16 inputs
(the tolerance the benchmark definition states), tighter where the math allows.
"""
import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ops(pkg, lib):
    assert torch.cuda.is_available(), "GPU tests need an MI355X"
    return pkg.ops


def _close(a, b, rtol=RTOL, atol=ATOL):
    a, b = a.float().cpu(), b.float().cpu()
    ok = torch.allclose(a, b, rtol=rtol, atol=atol)
    if not ok:
        d = (a - b).abs()
        _say("max abs diff", d.max().item(), "at", np.unravel_index(d.argmax().item(), a.shape),
             "ref scale", b.abs().max().item(), "frac bad",
             (d > atol + rtol * b.abs()).float().mean().item())
    return ok


# ------------------------------------------------------------------------------- routing
@pytest.mark.parametrize("T,E,k,dtype,quant", [
    (2048, 8, 2, torch.bfloat16, False), (4096, 64, 8, torch.bfloat16, False),
    (1000, 64, 8, torch.float32, False), (777, 128, 8, torch.bfloat16, False),
    (300, 200, 5, torch.float32, True), (128, 512, 64, torch.bfloat16, False),
    (64, 8, 8, torch.float32, True), (513, 3, 1, torch.bfloat16, True), (1, 64, 8, torch.float32, False),
])
def test_router_topk_bit_exact(ops, T, E, k, dtype, quant):
    _say("router_topk", T, E, k, dtype, quant)
    g = torch.Generator().manual_seed(T + E + k)
    logits = torch.randn(T, E, generator=g)
    if quant:
        logits = (logits * 2).round() / 2  # many exact ties, including across the k-th boundary
        logits[0, :] = 0.0
    logits = logits.to(dtype)
    ids, gates = ops.router_topk(logits.cuda(), k)
    oid, osel = O.topk_select(logits, k)
    assert np.array_equal(ids.cpu().numpy().reshape(T, k), oid.astype(np.int32))
    og = O.gates_from_selected(osel)
    assert torch.allclose(gates.cpu().reshape(T, k), og, atol=1e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_topk_non_finite_logits(ops, dtype):
    """Experts masked with -inf (fewer finite logits than k included), a +inf logit, a row of
    -inf and a NaN: selection and gates as torch.topk + softmax give them (mlp.py:101-102) --
    masked experts are taken last, lowest index first, with gate 0; a row whose softmax is
    NaN in the reference is NaN here; ids stay distinct and in range; other rows are untouched."""
    T, E, k = 256, 64, 8
    g = torch.Generator().manual_seed(77)
    logits = torch.randn(T, E, generator=g)
    inf = float("inf")
    logits[0, 5:] = -inf                       # 5 finite logits, k = 8
    logits[1, ::2] = -inf                      # half of the experts masked
    logits[2, 17] = inf
    logits[3, :] = -inf
    logits[4, 9] = float("nan")
    logits[5, :] = 0.0
    logits[5, 60:] = -inf
    clean = logits.clone()
    logits = logits.to(dtype)
    ids, gates = ops.router_topk(logits.cuda(), k)
    ids = ids.cpu().numpy().reshape(T, k)
    gates = gates.cpu().reshape(T, k)
    assert ids.min() >= 0 and ids.max() < E
    assert all(len(set(row)) == k for row in ids)
    oid, osel = O.topk_select(logits, k)
    assert np.array_equal(ids, oid.astype(np.int32))
    og = O.gates_from_selected(osel)
    assert torch.allclose(gates, og, atol=1e-6, rtol=1e-5, equal_nan=True)
    assert torch.isnan(gates[2]).all() and torch.isnan(gates[3]).all() and torch.isnan(gates[4]).all()
    assert ids[4, 0] == 9                      # a NaN ranks above every number, as for torch.topk,
    #                                            whatever its sign (torch's CPU cast to bf16 sets it)
    assert torch.equal(gates[0, 5:], torch.zeros(3)) and sorted(ids[0, :5]) == [0, 1, 2, 3, 4]
    assert list(ids[0, 5:]) == [5, 6, 7]
    assert torch.isfinite(gates[6:]).all()
    # the library routine on the rows where it is unambiguous (no ties among the selected)
    if dtype == torch.float32:                 # (bf16 rows hold ties, which the library orders its own way)
        assert np.array_equal(ids[6:], torch.topk(clean[6:], k).indices.numpy())


def test_router_topk_with_bias(ops):
    T, E, k = 4096, 8, 2
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(T, E, generator=g).to(torch.bfloat16)
    bias = -1.2 * torch.log(torch.randperm(E, generator=g).float() + 1)
    ids, gates = ops.router_topk(logits.cuda(), k, bias.cuda())
    biased = logits.float() + bias  # the same fp32 add the kernel does
    oid, osel = O.topk_select(biased, k)
    assert np.array_equal(ids.cpu().numpy().reshape(T, k), oid.astype(np.int32))
    assert torch.allclose(gates.cpu().reshape(T, k), O.gates_from_selected(osel), atol=1e-6, rtol=1e-5)
    counts = np.bincount(oid.reshape(-1), minlength=E)
    assert counts.max() > 3 * counts.min()  # the bias really skews the load


def test_router_topk_bwd(ops):
    T, E, k = 512, 64, 8
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(T, E, generator=g)
    dgates = torch.randn(T * k, generator=g)
    ids, gates = ops.router_topk(logits.cuda(), k)
    dl = ops.router_topk_bwd(gates, dgates.cuda(), ids, T, E, k, torch.float32).cpu()
    lg = logits.clone().requires_grad_(True)
    sel = torch.gather(lg, 1, ids.cpu().long().reshape(T, k))
    (torch.softmax(sel, -1).reshape(-1) * dgates).sum().backward()
    assert torch.allclose(dl, lg.grad, atol=1e-6, rtol=1e-4)
    assert (dl != 0).sum(1).max() <= k
    dlb = ops.router_topk_bwd(gates, dgates.cuda(), ids, T, E, k, torch.bfloat16).cpu()
    assert torch.equal(dlb, dl.to(torch.bfloat16))


# ------------------------------------------------------------------------------- dispatch
def _ids_case(name, rng):
    if name == "uniform":
        return rng.integers(0, 64, size=131072), 64
    if name == "ragged":
        return rng.integers(0, 7, size=1000), 7
    if name == "one_expert":
        return np.zeros(555, dtype=np.int64), 1
    if name == "all_same_of_many":
        return np.full(300, 5, dtype=np.int64), 9
    if name == "empty_experts":
        ids = rng.integers(0, 16, size=5000)
        ids[ids == 3] = 4
        ids[ids == 15] = 0
        return ids, 16
    if name == "tiny":
        return np.array([2, 0, 2, 1, 0, 2]), 3
    if name == "max_experts":
        return rng.integers(0, 512, size=70000), 512
    if name == "skewed":
        p = rng.dirichlet(np.full(16, 0.3))
        return rng.choice(16, size=32768, p=p), 16
    if name == "zero_rows":
        return np.zeros(0, dtype=np.int64), 4
    raise KeyError(name)


@pytest.mark.parametrize("case", ["uniform", "ragged", "one_expert", "all_same_of_many",
                                  "empty_experts", "tiny", "max_experts", "skewed", "zero_rows"])
def test_histogram_scan_bit_exact(ops, case):
    _say("histogram_scan", case)
    ids, E = _ids_case(case, np.random.default_rng(7))
    d = torch.from_numpy(ids.astype(np.int32)).cuda()
    counts, offs, p2r, r2p = ops.histogram_scan(d, E)
    oc, ostarts = O.counts_offsets(ids, E)
    op2r, or2p = O.stable_permutation(ids)
    assert np.array_equal(counts.cpu().numpy(), oc.astype(np.int32))
    assert np.array_equal(offs.cpu().numpy(), ostarts)
    assert np.array_equal(p2r.cpu().numpy(), op2r.astype(np.int32))
    assert np.array_equal(r2p.cpu().numpy(), or2p.astype(np.int32))


def test_dispatch_and_routing_on_random_sizes(ops):
    """Forty seeded random sizes through the integer kernels -- row counts around the 64-lane and
    256-row block edges, 1 to 512 experts, skewed and uniform draws -- all bit-exact against
    numpy; and the same number of random routing problems (E up to 512, k up to 64, both logit
    dtypes, with and without quantised ties)."""
    rng = np.random.default_rng(4242)
    for case in range(40):
        E = int(rng.choice([1, 2, 3, int(rng.integers(4, 65)), int(rng.integers(65, 513))]))
        R = int(rng.choice([rng.integers(1, 70), rng.integers(250, 262), rng.integers(1000, 40000)]))
        if rng.random() < 0.5:
            ids = rng.integers(0, E, size=R)
        else:
            ids = rng.choice(E, size=R, p=rng.dirichlet(np.full(E, 0.2)))
        _say("random dispatch", case, "R", R, "E", E)
        counts, offs, p2r, r2p = ops.histogram_scan(torch.from_numpy(ids.astype(np.int32)).cuda(), E)
        oc, ostarts = O.counts_offsets(ids, E)
        op2r, or2p = O.stable_permutation(ids)
        assert np.array_equal(counts.cpu().numpy(), oc.astype(np.int32)), (case, R, E)
        assert np.array_equal(offs.cpu().numpy(), ostarts), (case, R, E)
        assert np.array_equal(p2r.cpu().numpy(), op2r.astype(np.int32)), (case, R, E)
        assert np.array_equal(r2p.cpu().numpy(), or2p.astype(np.int32)), (case, R, E)
    g = torch.Generator().manual_seed(4243)
    for case in range(40):
        E = int(rng.choice([1, 2, 5, int(rng.integers(6, 65)), int(rng.integers(65, 513))]))
        k = int(rng.integers(1, min(E, 64) + 1))
        T = int(rng.choice([1, 3, int(rng.integers(4, 300)), int(rng.integers(300, 5000))]))
        dtype = torch.bfloat16 if rng.random() < 0.5 else torch.float32
        logits = torch.randn(T, E, generator=g)
        if rng.random() < 0.4:
            logits = (logits * 2).round() / 2
        logits = logits.to(dtype)
        _say("random routing", case, "T", T, "E", E, "k", k, dtype)
        ids, gates = ops.router_topk(logits.cuda(), k)
        oid, osel = O.topk_select(logits, k)
        assert np.array_equal(ids.cpu().numpy().reshape(T, k), oid.astype(np.int32)), (case, T, E, k)
        assert torch.allclose(gates.cpu().reshape(T, k), O.gates_from_selected(osel), atol=1e-6, rtol=1e-5)


def test_histogram_scan_counts_ids_out_of_range(pkg, ops):
    """Expert ids outside [0, E): counted on the device, rows placed with the nearest valid
    expert (the result equals the sort of the clipped ids), nothing read or written out of
    bounds; valid inputs report zero.  `experts_rows(check_ids=True)` turns the count into an
    exception."""
    _say("histogram_scan with invalid ids")
    rng = np.random.default_rng(11)
    E, R = 12, 3000
    ids = rng.integers(0, E, size=R)
    where = rng.choice(R, size=37, replace=False)
    ids[where[:20]] = rng.integers(E, E + 1000, size=20)
    ids[where[20:]] = -rng.integers(1, 1000, size=17)
    d = torch.from_numpy(ids.astype(np.int32)).cuda()
    counts, offs, p2r, r2p, bad = ops.histogram_scan(d, E, return_bad=True)
    assert bad.item() == 37
    clipped = np.clip(ids, 0, E - 1)
    oc, ostarts = O.counts_offsets(clipped, E)
    op2r, or2p = O.stable_permutation(clipped)
    assert np.array_equal(counts.cpu().numpy(), oc.astype(np.int32))
    assert np.array_equal(offs.cpu().numpy(), ostarts)
    assert np.array_equal(p2r.cpu().numpy(), op2r.astype(np.int32))
    assert np.array_equal(r2p.cpu().numpy(), or2p.astype(np.int32))
    good = torch.from_numpy(clipped.astype(np.int32)).cuda()
    assert ops.histogram_scan(good, E, return_bad=True)[4].item() == 0
    assert ops.histogram_scan(good[:0], E, return_bad=True)[4].item() == 0
    H, I = 64, 32
    g = torch.Generator().manual_seed(3)
    rows = torch.randn(R, H, generator=g).to(torch.bfloat16).cuda()
    ws = [(torch.randn(*s_, generator=g) * 0.1).to(torch.bfloat16).cuda() for s_ in ((E, I, H), (E, I, H), (E, H, I))]
    out, rt = pkg.experts_rows(rows, good, *ws, return_routing=True, check_ids=True)
    assert rt["bad_ids"].item() == 0
    with pytest.raises(ValueError, match="37 of 3000"):
        pkg.experts_rows(rows, d, *ws, check_ids=True)
    out_bad, rt = pkg.experts_rows(rows, d, *ws, return_routing=True)   # unchecked: runs, and says so
    assert rt["bad_ids"].item() == 37 and torch.equal(out_bad, out)


def _random_mover_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        E = int(rng.integers(1, 70))
        k = int(rng.integers(1, min(E, 9) + 1))
        out.append((int(rng.integers(1, 400)), int(rng.choice([rng.integers(1, 40), rng.integers(40, 600)])) * 8, k, E))
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,H,k,E", [(300, 256, 2, 8), (64, 2048, 8, 64), (5, 8, 1, 3), (33, 1032, 3, 5),
                                     (17, 4096, 2, 4)] + _random_mover_shapes(8, 99))
def test_permute_and_combine(ops, dtype, T, H, k, E):
    _say("permute/combine", dtype, T, H, k, E)
    g = torch.Generator().manual_seed(T + H)
    rng = np.random.default_rng(T)
    x = torch.randn(T, H, generator=g).to(dtype)
    ids = np.stack([rng.permutation(E)[:k] for _ in range(T)]).reshape(-1)
    R = T * k
    _, _, p2r, r2p = ops.histogram_scan(torch.from_numpy(ids.astype(np.int32)).cuda(), E)
    op2r, or2p = O.stable_permutation(ids)
    # permute fwd: pure copy (plus the fp32 -> bf16 rounding when x is fp32): bit-exact
    xp = ops.permute_fwd(x.cuda(), p2r, k).cpu()
    assert torch.equal(xp, x[torch.from_numpy(op2r // k)].to(torch.bfloat16))
    # the token-by-token variant (from the inverse map) writes the same rows
    assert torch.equal(ops.permute_fwd(x.cuda(), p2r, k, r2p).cpu(), xp)
    # combine fwd
    y = torch.randn(R, H, generator=g).to(torch.bfloat16)
    gates = torch.rand(R, generator=g)
    out = ops.combine_fwd(y.cuda(), gates.cuda(), r2p, T, k, dtype).cpu()
    ref = O.combine_rows(y.float(), gates, or2p, T, k)
    assert _close(out, ref, rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-2 if dtype == torch.bfloat16 else 1e-5)
    out2 = ops.combine_fwd(y.cuda(), gates.cuda(), r2p, T, k, dtype).cpu()
    assert torch.equal(out, out2)  # deterministic
    # un-gated k-sum (permute backward), with and without an addend
    dx = ops.permute_bwd(y.cuda(), r2p, T, k, dtype).cpu()
    ref = y.float()[torch.from_numpy(or2p)].view(T, k, H).sum(1)
    assert _close(dx, ref, rtol=1e-2 if dtype == torch.bfloat16 else 1e-6, atol=1e-2 if dtype == torch.bfloat16 else 1e-6)
    add = torch.randn(T, H, generator=g).to(dtype)
    dx = ops.permute_bwd(y.cuda(), r2p, T, k, dtype, addend=add.cuda()).cpu()
    assert _close(dx, ref + add.float(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-6, atol=2e-2 if dtype == torch.bfloat16 else 1e-6)
    # combine bwd
    dy = torch.randn(T, H, generator=g).to(dtype)
    dyp, dgates = ops.combine_bwd(dy.cuda(), y.cuda(), gates.cuda(), p2r, k)
    tok = torch.from_numpy(op2r // k)
    ref_dyp = (dy.float()[tok] * gates[torch.from_numpy(op2r)].unsqueeze(-1)).to(torch.bfloat16)
    assert torch.equal(dyp.cpu(), ref_dyp)  # one fp32 multiply then one rounding: bit-exact
    ref_dg = torch.empty(R)
    ref_dg[torch.from_numpy(op2r)] = (dy.float()[tok] * y.float()).sum(-1)
    assert torch.allclose(dgates.cpu(), ref_dg, rtol=1e-4, atol=1e-3)
    # the token-by-token variant: same bits
    dyp_t, dgates_t = ops.combine_bwd(dy.cuda(), y.cuda(), gates.cuda(), p2r, k, r2p)
    assert torch.equal(dyp_t, dyp) and torch.equal(dgates_t, dgates)
    # gate-less variant (post-dispatch entry): pure row permutation both ways
    dyp2, none = ops.combine_bwd(dy.cuda(), None, None, p2r, k)
    assert none is None and torch.equal(dyp2.cpu(), dy[tok].to(torch.bfloat16))
    dyp3, none = ops.combine_bwd(dy.cuda(), None, None, p2r, k, r2p)
    assert none is None and torch.equal(dyp3, dyp2)


def test_cast(ops):
    g = torch.Generator().manual_seed(9)
    for n in (1, 7, 8, 1000, 1 << 20, (1 << 20) + 3):
        w = torch.randn(n, generator=g)
        assert torch.equal(ops.cast_bf16(w.cuda()).cpu(), w.to(torch.bfloat16))


# ------------------------------------------------------------------------------- GEMMs
def _gemm_case(R, H, I, E, seed, empty=(), std=0.05):
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    live = np.array([e for e in range(E) if e not in empty])
    ids = np.sort(live[rng.integers(0, len(live), size=R)])
    counts, starts = O.counts_offsets(ids, E)
    xp = torch.randn(R, H, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(E, I, H, generator=g) * std).to(torch.bfloat16)
    w3 = (torch.randn(E, I, H, generator=g) * std).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, generator=g) * std).to(torch.bfloat16)
    return xp, w1, w3, w2, starts


GEMM_SHAPES = [
    # R, H, I, E, empty experts
    (1000, 256, 128, 5, ()),        # ragged tails in every expert
    (4096, 1024, 512, 8, ()),       # config-1 shape
    (777, 200, 72, 7, (2, 5)),      # H, I not multiples of the tile; empty experts
    (130, 64, 64, 16, (0, 15)),     # experts with a handful of rows
    (2048, 128, 320, 1, ()),        # single expert
]


def _random_gemm_shapes(n, seed):
    """Seeded random shapes: row counts around the 256-row tile edges, widths that are multiples
    of 8 only, expert counts from 1 to 24 with a random subset left without rows."""
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        E = int(rng.integers(1, 25))
        R = int(rng.choice([rng.integers(1, 64), rng.integers(200, 330), rng.integers(500, 3000)]))
        H = int(rng.integers(1, 76)) * 8
        I = int(rng.integers(1, 76)) * 8
        empty = tuple(int(e) for e in rng.choice(E, size=int(rng.integers(0, max(1, E // 3) + 1)), replace=False)) if E > 1 else ()
        if len(empty) == E:
            empty = empty[1:]
        out.append((R, H, I, E, tuple(sorted(empty))))
    return out


@pytest.mark.parametrize("R,H,I,E,empty", GEMM_SHAPES + _random_gemm_shapes(12, 2024))
def test_expert_gemms_forward_backward(ops, R, H, I, E, empty):
    _say("gemm", R, H, I, E, empty)
    xp, w1, w3, w2, starts = _gemm_case(R, H, I, E, seed=R + H, empty=empty)
    offs = torch.from_numpy(starts).cuda()
    f = O.expert_ffn_rows(xp.float(), starts, w1.float(), w3.float(), w2.float())
    g, u, act = ops.gemm_gateup(xp.cuda(), w1.cuda(), w3.cuda(), offs, save_gu=True)
    assert _close(g, f["g"]) and _close(u, f["u"]) and _close(act, f["act"])
    _, _, act_only = ops.gemm_gateup(xp.cuda(), w1.cuda(), w3.cuda(), offs, save_gu=False)
    assert torch.equal(act_only, act)
    y = ops.gemm_down(act, w2.cuda(), offs)
    af = act.float().cpu()
    ref_y = torch.zeros(R, H)
    for e in range(E):
        a, b = int(starts[e]), int(starts[e + 1])
        ref_y[a:b] = af[a:b] @ w2[e].float().t()
    assert _close(y, ref_y)  # down projection alone, fed the device's own act
    assert _close(y, O.expert_ffn_rows(xp.float(), starts, w1.float(), w3.float(), w2.float(), emulate_bf16=True)["y"])

    # backward pieces, each fed the device's own (bf16) forward tensors so that one
    # kernel is checked at a time
    gen = torch.Generator().manual_seed(1)
    dyp = torch.randn(R, H, generator=gen).to(torch.bfloat16)
    gf, uf, af = g.float().cpu(), u.float().cpu(), act.float().cpu()
    dg, du = ops.gemm_dgrad_down(dyp.cuda(), w2.cuda(), g, u, offs)
    ref_dg, ref_du = torch.zeros(R, I), torch.zeros(R, I)
    ref_dw2 = torch.zeros(E, H, I)
    for e in range(E):
        a, b = int(starts[e]), int(starts[e + 1])
        dact = dyp[a:b].float() @ w2[e].float()
        s = torch.sigmoid(gf[a:b])
        ref_dg[a:b] = dact * uf[a:b] * (s * (1 + gf[a:b] * (1 - s)))
        ref_du[a:b] = dact * gf[a:b] * s
        ref_dw2[e] = dyp[a:b].float().t() @ af[a:b]
    assert _close(dg, ref_dg) and _close(du, ref_du)
    # g and u in the library's blocked layout (what the autograd functions save): the forward's
    # act and every result of the backward kernel must be the same bits as with [R, I] rows,
    # separate or side by side, with and without the gate gradients' block sums
    gu, act_b = ops.gemm_gateup_blocked(xp.cuda(), w1.cuda(), w3.cuda(), offs)
    assert torch.equal(act_b, act)
    dg_r, du_r, part_r = ops.gemm_dgrad_down(dyp.cuda(), w2.cuda(), g, u, offs, dgate_blocks=True)
    assert torch.equal(dg_r, dg) and torch.equal(du_r, du)
    dg_b, du_b, part_b = ops.gemm_dgrad_down_blocked(dyp.cuda(), w2.cuda(), gu, offs, dgate_blocks=True)
    assert torch.equal(dg_b, dg) and torch.equal(du_b, du)
    assert torch.equal(part_b.view(torch.int32), part_r.view(torch.int32))
    dg_b2, du_b2, none = ops.gemm_dgrad_down_blocked(dyp.cuda(), w2.cuda(), gu, offs)
    assert none is None and torch.equal(dg_b2, dg) and torch.equal(du_b2, du)
    dgu_b, part_b3 = ops.gemm_dgrad_down_blocked(dyp.cuda(), w2.cuda(), gu, offs, dgate_blocks=True, packed=True)
    assert torch.equal(dgu_b[:, :I], dg) and torch.equal(dgu_b[:, I:], du)
    assert torch.equal(part_b3.view(torch.int32), part_r.view(torch.int32))
    dxp = ops.gemm_dgrad_gateup(dg, du, w1.cuda(), w3.cuda(), offs)
    # both row-tile heights of the four row-ragged products, forced in turn (the automatic choice
    # above took one of them from the shape): the same bits on every output
    L = ops._lib.load()
    try:
        for rows in (128, 256):
            L.cdll.moe_gemm_force_row_tile(rows)
            g_t, u_t, act_t = ops.gemm_gateup(xp.cuda(), w1.cuda(), w3.cuda(), offs, save_gu=True)
            assert torch.equal(g_t, g) and torch.equal(u_t, u) and torch.equal(act_t, act), rows
            assert torch.equal(ops.gemm_down(act, w2.cuda(), offs), y), rows
            gu_t, act_t = ops.gemm_gateup_blocked(xp.cuda(), w1.cuda(), w3.cuda(), offs)
            dg_t, du_t, part_t = ops.gemm_dgrad_down_blocked(dyp.cuda(), w2.cuda(), gu_t, offs, dgate_blocks=True)
            assert torch.equal(act_t, act) and torch.equal(dg_t, dg) and torch.equal(du_t, du), rows
            assert torch.equal(part_t.view(torch.int32), part_r.view(torch.int32)), rows
            dg_t, du_t = ops.gemm_dgrad_down(dyp.cuda(), w2.cuda(), g, u, offs)
            assert torch.equal(dg_t, dg) and torch.equal(du_t, du), rows
            assert torch.equal(ops.gemm_dgrad_gateup(dg, du, w1.cuda(), w3.cuda(), offs), dxp), rows
    finally:
        L.cdll.moe_gemm_force_row_tile(0)
    dgf, duf = dg.float().cpu(), du.float().cpu()
    ref_dxp = torch.zeros(R, H)
    ref_dw1, ref_dw3 = torch.zeros(E, I, H), torch.zeros(E, I, H)
    for e in range(E):
        a, b = int(starts[e]), int(starts[e + 1])
        ref_dxp[a:b] = dgf[a:b] @ w1[e].float() + duf[a:b] @ w3[e].float()
        ref_dw1[e] = dgf[a:b].t() @ xp[a:b].float()
        ref_dw3[e] = duf[a:b].t() @ xp[a:b].float()
    assert _close(dxp, ref_dxp)
    for dt in (torch.float32, torch.bfloat16):
        scale = 1.0 if dt == torch.float32 else 1.0
        dw2 = ops.gemm_wgrad(dyp.cuda(), act, offs, E, dt)
        dw1 = ops.gemm_wgrad(dg, xp.cuda(), offs, E, dt)
        dw3 = ops.gemm_wgrad(du, xp.cuda(), offs, E, dt)
        assert _close(dw2, ref_dw2) and _close(dw1, ref_dw1) and _close(dw3, ref_dw3)
        for e in empty:
            assert not dw1[e].any() and not dw2[e].any() and not dw3[e].any()
    # accumulate into an existing fp32 gradient; deterministic across runs
    base = torch.randn(E, H, I, generator=gen)
    acc = ops.gemm_wgrad(dyp.cuda(), act, offs, E, torch.float32, out=base.clone().cuda())
    assert _close(acc, ref_dw2 + base)
    again = ops.gemm_wgrad(dyp.cuda(), act, offs, E, torch.float32)
    assert torch.equal(again, ops.gemm_wgrad(dyp.cuda(), act, offs, E, torch.float32))
    # the contraction cut into S row segments per expert (what the autograd functions do when
    # the output has too few tiles to fill the chip): exact segment bounds, same sums up to
    # fp32 rounding, experts without rows still exactly zero
    for S in (2, 5):
        seg = ops.segment_offsets(offs, E, S)
        o = offs.cpu().numpy().astype(np.int64)
        want = [o[e] + (o[e + 1] - o[e]) * s_ // S for e in range(E) for s_ in range(S)] + [o[E]]
        assert seg.cpu().tolist() == [int(v) for v in want]
        part = ops.gemm_wgrad(dyp.cuda(), act, seg, E * S, torch.float32).view(E, S, H, I).sum(1)
        assert torch.allclose(part, again, rtol=1e-4, atol=1e-4 * float(again.abs().max()))
        for e in empty:
            assert not part[e].any()
    # segments of bounded length (what the autograd functions use): exact bounds against numpy,
    # the fixed-order reduction against the unsplit product, fresh and accumulating, both dtypes
    for Lseg in (64, 200, 4096):
        seg, seg_start, S_max = ops.segment_offsets_by_length(offs, E, Lseg, R)
        o = offs.cpu().numpy().astype(np.int64)
        n = o[1:] - o[:-1]
        ns = -(-n // Lseg)
        assert S_max == -(-R // Lseg) + E and ns.sum() <= S_max
        assert seg_start.cpu().tolist() == [0] + np.cumsum(ns).tolist()
        want = [int(o[e] + n[e] * j // ns[e]) for e in range(E) for j in range(ns[e])]
        want += [int(o[E])] * (S_max + 1 - len(want))
        assert seg.cpu().tolist() == want
        if S_max > 1024:
            continue
        part = ops.gemm_wgrad(dyp.cuda(), act, seg, S_max, torch.float32)
        red = ops.wgrad_reduce_segments(part, seg_start, E, torch.float32)
        assert torch.allclose(red, again, rtol=1e-4, atol=1e-4 * float(again.abs().max()))
        assert torch.equal(red, ops.wgrad_reduce_segments(part, seg_start, E, torch.float32))
        for e in empty:
            assert not red[e].any()
        red16 = ops.wgrad_reduce_segments(part, seg_start, E, torch.bfloat16)
        assert torch.equal(red16, red.to(torch.bfloat16))
        acc2 = ops.wgrad_reduce_segments(part, seg_start, E, torch.float32, out=base.clone().cuda())
        assert torch.allclose(acc2, red + base.cuda(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("R,H,I,E,empty", [(1000, 256, 128, 5, ()), (777, 200, 72, 7, (2, 5)),
                                           (3000, 512, 1024, 4, ())])
def test_gate_gradients_from_the_dgrad_down_kernel(ops, R, H, I, E, empty):
    """The gate gradient <dy[token], y[row]> without reading y: the dgrad-down kernel leaves
    per-row block sums of <dact, act>, which add up to gate * <dy, y> because its input rows are
    gate * dy.  Checked against the direct product (and against the kernel that does read y)."""
    _say("gate gradients via dgrad-down", R, H, I, E, empty)
    xp, w1, w3, w2, starts = _gemm_case(R, H, I, E, seed=R + I, empty=empty)
    offs = torch.from_numpy(starts).cuda()
    gen = torch.Generator().manual_seed(R)
    k = 1  # every row its own "token": row_to_pos is then any permutation
    perm = torch.randperm(R, generator=gen).to(torch.int32)           # row_to_pos
    inv = torch.empty_like(perm)
    inv[perm.long()] = torch.arange(R, dtype=torch.int32)             # pos_to_row
    gates = (torch.rand(R, generator=gen) * 0.9 + 0.05)
    gates[::97] = 0.0  # underflowed gates: gradient defined as 0
    dy = torch.randn(R, H, generator=gen).to(torch.bfloat16)
    g, u, act = ops.gemm_gateup(xp.cuda(), w1.cuda(), w3.cuda(), offs, save_gu=True)
    y = ops.gemm_down(act, w2.cuda(), offs)
    dyp, dgates_direct = ops.combine_bwd(dy.cuda(), y, gates.cuda(), inv.cuda(), k)
    dg0, du0 = ops.gemm_dgrad_down(dyp, w2.cuda(), g, u, offs)
    dg, du, part = ops.gemm_dgrad_down(dyp, w2.cuda(), g, u, offs, dgate_blocks=True)
    assert torch.equal(dg, dg0) and torch.equal(du, du0)
    assert part.shape == (((I + 255) // 256) * 4, R) and torch.isfinite(part).all()
    dgates = ops.dgates_from_blocks(part, gates.cuda(), perm.cuda()).cpu()
    # reference in fp32 on the CPU: <dy[r], y_fp32[pos(r)]> with y from the bf16 act the device made
    af = act.float().cpu()
    yf = torch.zeros(R, H)
    for e in range(E):
        a, b = int(starts[e]), int(starts[e + 1])
        yf[a:b] = af[a:b] @ w2[e].float().t()
    ref = (dy.float() * yf[perm.long()]).sum(-1)
    live = gates != 0
    assert torch.equal(dgates[~live], torch.zeros(int((~live).sum())))
    scale = ref[live].abs().max().item()
    assert torch.allclose(dgates[live], ref[live], rtol=2e-2, atol=2e-2 * scale), \
        (dgates[live] - ref[live]).abs().max().item() / scale
    # and the two device routes agree to the same bar
    d2 = dgates_direct.cpu()
    assert torch.allclose(dgates[live], d2[live], rtol=2e-2, atol=2e-2 * scale)
    again = ops.dgates_from_blocks(ops.gemm_dgrad_down(dyp, w2.cuda(), g, u, offs, dgate_blocks=True)[2],
                                   gates.cuda(), perm.cuda()).cpu()
    assert torch.equal(again, dgates)  # reproducible
    # the walk by position (coalesced block reads, scattered results): the same bits
    by_pos = ops.dgates_from_blocks(part, gates.cuda(), perm.cuda(), inv.cuda()).cpu()
    assert torch.equal(by_pos, dgates)


@pytest.mark.parametrize("R,H,I,E,empty", [(1000, 256, 256, 5, ()), (3000, 520, 512, 7, (2, 5)), (8192, 1024, 1024, 8, ()),
                                           (130, 64, 256, 16, (0, 15))])
def test_packed_row_gradients_and_paired_weight_gradients(pkg, ops, R, H, I, E, empty):
    """dg and du side by side in one buffer and both their weight gradients from one launch:
    the same bits as the separate kernels (same tiles, same order of additions), with fp32 and
    bf16 results, with accumulation, and with the gate gradients' block sums."""
    _say("packed dg|du and paired wgrad", R, H, I, E, empty)
    xp, w1, w3, w2, starts = _gemm_case(R, H, I, E, seed=R + I + 1, empty=empty)
    offs = torch.from_numpy(starts).cuda()
    xp, w1, w3, w2 = xp.cuda(), w1.cuda(), w3.cuda(), w2.cuda()
    dyp = torch.randn(R, H, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).cuda()
    g, u, act = ops.gemm_gateup(xp, w1, w3, offs, save_gu=True)
    dg, du, part = ops.gemm_dgrad_down(dyp, w2, g, u, offs, dgate_blocks=True)
    dgu, part2 = ops.gemm_dgrad_down_packed(dyp, w2, g, u, offs, dgate_blocks=True)
    assert dgu.shape == (R, 2 * I)
    assert torch.equal(dgu[:, :I], dg) and torch.equal(dgu[:, I:], du) and torch.equal(part2, part)
    dgu3, none = ops.gemm_dgrad_down_packed(dyp, w2, g, u, offs)
    assert none is None and torch.equal(dgu3, dgu)
    assert torch.equal(ops.gemm_dgrad_gateup_packed(dgu, w1, w3, offs), ops.gemm_dgrad_gateup(dg, du, w1, w3, offs))
    for dt in (torch.float32, torch.bfloat16):
        a1, a3 = ops.gemm_wgrad_pair(dgu, xp, offs, E, dt)
        b1, b3 = ops.gemm_wgrad(dg, xp, offs, E, dt), ops.gemm_wgrad(du, xp, offs, E, dt)
        assert torch.equal(a1, b1) and torch.equal(a3, b3)
        ops.gemm_wgrad_pair(dgu, xp, offs, E, dt, out1=a1, out3=a3)        # accumulate into the results
        ops.gemm_wgrad(dg, xp, offs, E, dt, out=b1)
        ops.gemm_wgrad(du, xp, offs, E, dt, out=b3)
        assert torch.equal(a1, b1) and torch.equal(a3, b3)
        for e in empty:
            assert not a1[e].any() and not a3[e].any()
    if I == 256:  # a width whose 256-row tiles would straddle the halves is refused
        with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_SHAPE"):
            ops.gemm_wgrad_pair(dgu[:, :2 * 136].contiguous(), xp, offs, E, torch.float32)


def test_grouped_gemms_on_buffers_beyond_4_gib(ops):
    """Row buffers larger than 4 GiB, one expert owning more than 4 GiB of them: the rows on
    both sides of the 2^32-byte mark (row 2^20 at 4096 bytes per row) and the last rows must come
    out as they do at the start of the buffer, for every grouped product."""
    _say("grouped GEMMs, R*H*2 > 2^32")
    H, I, E = 2048, 16, 3
    n0 = (1 << 20) + 2000
    R = n0 + 900
    offs = torch.tensor([0, n0, n0, R], dtype=torch.int32).cuda()   # expert 1 has no rows
    gen = torch.Generator(device="cuda").manual_seed(5)
    xp = torch.randn(R, H, device="cuda", generator=gen).to(torch.bfloat16)
    assert xp.numel() * 2 > 1 << 32
    w1 = (torch.randn(E, I, H, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    w3 = (torch.randn(E, I, H, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn(E, H, I, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    windows = [(0, 300), ((1 << 20) - 300, (1 << 20) + 300), (n0 - 200, n0), (n0, n0 + 200), (R - 150, R)]
    expert_of = lambda a: 0 if a < n0 else 2

    g, u, act = ops.gemm_gateup(xp, w1, w3, offs, save_gu=True)
    y = ops.gemm_down(act, w2, offs)
    dg, du = ops.gemm_dgrad_down(xp, w2, g, u, offs)          # xp doubles as the incoming gradient rows
    dxp = ops.gemm_dgrad_gateup(dg, du, w1, w3, offs)
    for a, b in windows:
        e = expert_of(a)
        xs = xp[a:b].float()
        gr, ur = xs @ w1[e].float().t(), xs @ w3[e].float().t()
        assert _close(g[a:b], gr) and _close(u[a:b], ur) and _close(act[a:b], torch.nn.functional.silu(gr) * ur), (a, b)
        assert _close(y[a:b], act[a:b].float() @ w2[e].float().t()), (a, b)
        dact = xs @ w2[e].float()
        gf, uf = g[a:b].float(), u[a:b].float()
        sg = torch.sigmoid(gf)
        assert _close(dg[a:b], dact * uf * (sg * (1 + gf * (1 - sg)))) and _close(du[a:b], dact * gf * sg), (a, b)
        assert _close(dxp[a:b], dg[a:b].float() @ w1[e].float() + du[a:b].float() @ w3[e].float()), (a, b)
    # weight gradient: a contraction that runs across the 4 GiB mark (fixed order, fp32 sums)
    dw = ops.gemm_wgrad(act, xp, offs, E, torch.float32)        # [E, I, H]
    for e, (a, b) in ((0, (0, n0)), (2, (n0, R))):
        ref = torch.zeros(I, H, device="cuda")
        for c in range(a, b, 1 << 18):
            d = min(b, c + (1 << 18))
            ref += act[c:d].float().t() @ xp[c:d].float()
        rel = ((dw[e] - ref).norm() / ref.norm()).item()
        _say(f"  dw[{e}] rel {rel:.2e}")
        assert rel < 1e-3
    assert not dw[1].any()


def test_gemm_zero_rows(ops):
    E, H, I = 4, 64, 32
    offs = torch.zeros(E + 1, dtype=torch.int32).cuda()
    xp = torch.empty(0, H, dtype=torch.bfloat16).cuda()
    w = torch.zeros(E, I, H, dtype=torch.bfloat16).cuda()
    g, u, act = ops.gemm_gateup(xp, w, w, offs, save_gu=True)
    assert act.shape == (0, I)
    dw = ops.gemm_wgrad(xp, act, offs, E, torch.float32)
    torch.cuda.synchronize()
    assert dw.shape == (E, H, I) and not dw.any()


def test_argument_checks_return_codes(pkg, ops):
    x = torch.zeros(4, 12, dtype=torch.bfloat16).cuda()  # H=12 is not a multiple of 8
    p2r = torch.zeros(4, dtype=torch.int32).cuda()
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_SHAPE"):
        ops.permute_fwd(x, p2r, 1)
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_LIMIT"):
        ops.router_topk(torch.zeros(2, 600).cuda(), 2)
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_SHAPE"):
        ops.router_topk(torch.zeros(2, 4).cuda(), 5)
    with pytest.raises(RuntimeError, match="GPU tensors"):
        ops.router_topk(torch.zeros(2, 4), 2)


def test_grouped_gemms_at_the_expert_limit(pkg, ops):
    """E = 1024, the most experts the grouped GEMMs take (their per-expert tile table lives in LDS):
    most experts empty, a few with ragged row counts, every bf16 mode and both fp32 GEMMs against
    per-expert products; E = 1025 is refused before anything is launched."""
    E, H, I = 1024, 64, 64
    g_ = torch.Generator().manual_seed(1024)
    counts = np.zeros(E, dtype=np.int64)
    for e, n in ((0, 300), (1, 1), (511, 257), (512, 64), (1022, 5), (1023, 129)):
        counts[e] = n
    offs_np = np.zeros(E + 1, dtype=np.int32)
    offs_np[1:] = np.cumsum(counts)
    R = int(offs_np[-1])
    offs = torch.from_numpy(offs_np).cuda()
    bf = torch.bfloat16
    xp = torch.randn(R, H, generator=g_).to(bf).cuda()
    dyp = torch.randn(R, H, generator=g_).to(bf).cuda()
    w1, w3 = ((torch.randn(E, I, H, generator=g_) * 0.2).to(bf).cuda() for _ in range(2))
    w2 = (torch.randn(E, H, I, generator=g_) * 0.2).to(bf).cuda()
    gg, uu, act = ops.gemm_gateup(xp, w1, w3, offs, save_gu=True)
    y = ops.gemm_down(act, w2, offs)
    dg, du = ops.gemm_dgrad_down(dyp, w2, gg, uu, offs)[:2]
    dxp = ops.gemm_dgrad_gateup(dg, du, w1, w3, offs)
    dw2 = ops.gemm_wgrad(dyp, act, offs, E, torch.float32)
    live = [e for e in range(E) if counts[e]]
    for e in live:
        a, b = int(offs_np[e]), int(offs_np[e + 1])
        xe = xp[a:b].float()
        ge, ue = xe @ w1[e].float().t(), xe @ w3[e].float().t()
        assert _close(gg[a:b], ge) and _close(uu[a:b], ue), e
        assert _close(act[a:b], torch.nn.functional.silu(ge) * ue), e
        assert _close(y[a:b], act[a:b].float() @ w2[e].float().t()), e
        assert _close(dxp[a:b], dg[a:b].float() @ w1[e].float() + du[a:b].float() @ w3[e].float()), e
        ref = dyp[a:b].float().t() @ act[a:b].float()
        assert ((dw2[e] - ref).norm() / ref.norm().clamp_min(1e-20)).item() < 1e-3, e
    dead = torch.tensor([e for e in range(E) if not counts[e]]).cuda()
    assert not dw2[dead].any()
    # the fp32 entries on the same offsets
    c32 = ops.f32_gemm_rows(xp.float(), w1.float(), offs, True)
    w32 = ops.f32_gemm_wgrad(dyp.float(), xp.float(), offs, E)
    for e in live:
        a, b = int(offs_np[e]), int(offs_np[e + 1])
        assert torch.allclose(c32[a:b], xp[a:b].float() @ w1[e].float().t(), rtol=1e-4, atol=1e-4), e
        assert torch.allclose(w32[e], dyp[a:b].float().t() @ xp[a:b].float(), rtol=1e-4, atol=1e-3), e
    assert not w32[dead].any()
    big = torch.zeros(1026, dtype=torch.int32).cuda()
    wbig = torch.zeros(1025, I, H, dtype=bf).cuda()
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_LIMIT"):
        ops.gemm_gateup(xp, wbig, wbig, big, save_gu=False)
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_LIMIT"):
        ops.f32_gemm_rows(xp.float(), wbig.float(), big, True)


@pytest.mark.parametrize("counts,M,N", [
    ([2700, 300], 4096, 2560),                    # 10 groups of 32 tiles for 8 XCDs, one expert with 90 % of the rows
    ([5, 0, 1900, 40, 0, 700, 64, 3], 2048, 1024),  # one group per expert, two experts empty
    ([300] * 7 + [2100], 1024, 2048),             # one heavy expert at the end of the list
])
def test_weight_gradient_under_skewed_routing(ops, counts, M, N):
    """The weight-gradient kernel deals its tiles to the XCDs longest first when the routing is
    skewed (at most 64 experts, whole groups of tiles per expert): every tile must still be
    computed exactly once, whichever workgroup gets it.  Checked against per-expert products,
    for both output dtypes and with accumulation."""
    _say("wgrad skew", counts, M, N)
    E, R = len(counts), int(sum(counts))
    offs_np = np.zeros(E + 1, dtype=np.int32)
    offs_np[1:] = np.cumsum(counts)
    offs = torch.from_numpy(offs_np).cuda()
    g_ = torch.Generator().manual_seed(M + N + E)
    a = torch.randn(R, M, generator=g_).to(torch.bfloat16).cuda()
    b = torch.randn(R, N, generator=g_).to(torch.bfloat16).cuda()
    dw = ops.gemm_wgrad(a, b, offs, E, torch.float32)
    dwb = ops.gemm_wgrad(a, b, offs, E, torch.bfloat16)
    prev = torch.randn(E, M, N, generator=g_).cuda()
    acc = prev.clone()
    ops.gemm_wgrad(a, b, offs, E, torch.float32, out=acc)
    for e in range(E):
        s, t = int(offs_np[e]), int(offs_np[e + 1])
        ref = a[s:t].float().t() @ b[s:t].float()
        if s == t:
            assert not dw[e].any() and not dwb[e].any() and torch.equal(acc[e], prev[e])
            continue
        assert ((dw[e] - ref).norm() / ref.norm()).item() < 1e-3, e
        assert ((dwb[e].float() - ref).norm() / ref.norm()).item() < 5e-3, e
        assert (((acc[e] - prev[e]) - ref).norm() / ref.norm()).item() < 1e-3, e
    dw2 = ops.gemm_wgrad(a, b, offs, E, torch.float32)
    assert torch.equal(dw, dw2)
