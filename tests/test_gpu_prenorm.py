"""The step before and the step after the layer, fused into it: the caller's RMSNorm
(model/modules/norm.py:14-19) writing the bf16 rows the layer consumes, the residual add
(model/gpt.py:33) riding in the combine kernel, and the three gradient streams into the
residual meeting in the normalisation's backward kernel.

The kernels are checked against the CPU restatement of the reference's norm (closed form,
torch autograd for the backward); the fused module call against the MoE oracle evaluated on
exactly the normalised rows and router logits the device produced."""
import pytest
import torch

from oracle import block_oracle as BO
from oracle import moe_oracle as O
from _tol import check

pytestmark = pytest.mark.gpu
EPS = 1e-6


def _say(*a):
    print(*a, flush=True)


def _norm_ref(x, w, bf16_in):
    """norm.py:14-19 on the CPU, including the cast back to the input dtype before the
    weight multiplies (fp32 weight times bf16 rows promotes to fp32)."""
    xf = x.float()
    n = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + EPS)
    if bf16_in:
        n = n.to(torch.bfloat16).float()
    return w.float() * n


@pytest.mark.parametrize("T,H,x_dt,d1_dt,use_d2,use_res", [
    (1, 256, torch.float32, torch.float32, True, True),
    (37, 2048, torch.float32, torch.float32, True, True),
    (300, 1024, torch.bfloat16, torch.bfloat16, True, True),
    (129, 4104, torch.float32, torch.bfloat16, False, True),   # 513 column groups: 4 per thread
    (2500, 512, torch.bfloat16, torch.float32, True, False),   # more rows than partial-sum blocks
    (64, 8192, torch.float32, torch.float32, False, False),
])
def test_rmsnorm_kernels(pkg, lib, T, H, x_dt, d1_dt, use_d2, use_res):
    ops = pkg.ops
    _say(f"rmsnorm kernels T={T} H={H} x {x_dt} d1 {d1_dt} d2={use_d2} dres={use_res}")
    g = torch.Generator().manual_seed(5 + T + H)
    x = (torch.randn(T, H, generator=g) * 1.7).to(x_dt)
    w = 1.0 + 0.2 * torch.randn(H, generator=g)
    d1 = torch.randn(T, H, generator=g).to(d1_dt)
    d2 = torch.randn(T, H, generator=g).to(torch.bfloat16) if use_d2 else None
    dres = torch.randn(T, H, generator=g).to(x_dt) if use_res else None
    cu = lambda t: None if t is None else t.cuda()

    xn, rstd = ops.rmsnorm_fwd(cu(x), cu(w), EPS)
    assert xn.dtype == torch.bfloat16 and rstd.dtype == torch.float32
    check("xn", xn, _norm_ref(x, w, x_dt == torch.bfloat16), say=_say)
    want_r = torch.rsqrt(x.float().pow(2).mean(-1) + EPS)
    assert torch.allclose(rstd.cpu(), want_r, rtol=1e-5, atol=0)

    dx, dw = ops.rmsnorm_bwd(cu(x), cu(w), rstd, cu(d1), cu(d2), cu(dres))
    assert dx.dtype == x_dt and dw.dtype == torch.float32 and dw.shape == (H,)
    xa = x.float().clone().requires_grad_(True)
    wa = w.clone().requires_grad_(True)
    gsum = d1.float() + (d2.float() if use_d2 else 0)
    BO.rmsnorm(xa, wa, EPS).backward(gsum)
    dx_ref = xa.grad + (dres.float() if use_res else 0)
    check("dx", dx, dx_ref, say=_say)
    check("dweight", dw, wa.grad, say=_say)
    # fixed reduction order: bit-identical on a second run
    dx2, dw2 = ops.rmsnorm_bwd(cu(x), cu(w), rstd, cu(d1), cu(d2), cu(dres))
    assert torch.equal(dx, dx2) and torch.equal(dw, dw2)


def test_rmsnorm_edges(pkg, lib):
    ops = pkg.ops
    w = torch.ones(64, device="cuda")
    xn, rstd = ops.rmsnorm_fwd(torch.empty(0, 64, device="cuda"), w, EPS)
    assert xn.shape == (0, 64) and rstd.shape == (0,)
    dx, dw = ops.rmsnorm_bwd(torch.empty(0, 64, device="cuda"), w, rstd, torch.empty(0, 64, device="cuda"))
    assert dx.shape == (0, 64) and torch.equal(dw, torch.zeros(64, device="cuda"))
    # an all-zero row normalises to zero (eps keeps the reciprocal finite)
    xn, rstd = ops.rmsnorm_fwd(torch.zeros(3, 64, device="cuda"), w, EPS)
    assert torch.equal(xn.float(), torch.zeros(3, 64, device="cuda")) and torch.isfinite(rstd).all()
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_LIMIT"):
        ops.rmsnorm_fwd(torch.zeros(2, 8200, device="cuda"), torch.ones(8200, device="cuda"), EPS)
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_SHAPE"):
        ops.rmsnorm_fwd(torch.zeros(2, 60, device="cuda"), torch.ones(60, device="cuda"), EPS)


def _fused_case(pkg, x_dt):
    cfg = pkg.ModelConfig(hidden_size=256, num_experts=8, num_experts_per_tok=2, moe_intermediate_size=128,
                          init_std=0.05)
    m = pkg.MoE(cfg, 2)
    from importlib import import_module
    norm = import_module(pkg.__name__ + ".block").RMSNorm(256, m.experts_gate_weights.device)
    g = torch.Generator().manual_seed(31)
    with torch.no_grad():
        norm.weight.copy_(1.0 + 0.2 * torch.randn(256, generator=g))
    B, T = 2, 160
    x = (torch.randn(B, T, 256, generator=g) * 1.3).to(x_dt).cuda().requires_grad_(True)
    dy = torch.randn(B, T, 256, generator=g).to(x_dt).cuda()
    return cfg, m, norm, x, dy, B, T


def test_fused_prenorm_module_matches_oracle(pkg, lib):
    _say("MoE.forward_prenorm: RMSNorm + layer + residual in one call, fp32 residual stream, bf16 autocast")
    cfg, m, norm, x, dy, B, T = _fused_case(pkg, torch.float32)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out, logits = m.forward_prenorm(x, norm)
    assert out.dtype == torch.float32 and out.shape == (B, T, 256)
    assert logits.dtype == torch.bfloat16 and logits.shape == (B, T, 8)
    out.backward(dy)
    names = ("experts_gate_weights", "experts_up_weights", "experts_down_weights")
    # the normalised rows the layer consumed (the kernel is deterministic: same bits again)
    xn, _ = pkg.ops.rmsnorm_fwd(x.detach().reshape(-1, 256), norm.weight.detach(), EPS)
    check("xn", xn, BO.rmsnorm(x.detach().cpu().reshape(-1, 256), norm.weight.detach().cpu(), EPS), say=_say)
    r = lambda t: t.detach().cpu().to(torch.bfloat16)
    wr, w1, w3, w2 = r(m.router.weight), *[r(getattr(m, n)) for n in names]
    lg = logits.detach().cpu().reshape(-1, 8)
    check("logits", lg, torch.nn.functional.linear(xn.cpu().float(), wr.float()), say=_say)
    f = O.moe_forward(xn.cpu(), wr, w1, w3, w2, 2, logits=lg)
    check("out", out.reshape(-1, 256), x.detach().cpu().reshape(-1, 256) + f["out"], say=_say)
    dyc = dy.cpu().reshape(-1, 256)
    b = O.moe_backward(f, dyc, wr, w1, w3, w2)
    fe = O.moe_forward(xn.cpu(), wr, w1, w3, w2, 2, logits=lg, emulate_bf16=True)
    be = O.moe_backward(fe, dyc, wr, w1, w3, w2, emulate_bf16=True)
    for n, key in zip(names + ("router.weight",), ("dw1", "dw3", "dw2", "dwr")):
        p = m.router.weight if key == "dwr" else getattr(m, n)
        assert p.grad is not None and p.grad.dtype == torch.float32
        check(key, p.grad, b[key], be[key], say=_say)
    # the gradient of the normalised rows goes back through the norm (torch autograd on the
    # CPU restatement) and meets the residual branch's gradient
    xa = x.detach().cpu().reshape(-1, 256).clone().requires_grad_(True)
    wa = norm.weight.detach().cpu().clone().requires_grad_(True)
    BO.rmsnorm(xa, wa, EPS).backward(b["dx"])
    check("dx", x.grad.reshape(-1, 256), dyc + xa.grad, say=_say)
    check("d norm.weight", norm.weight.grad, wa.grad, say=_say)


def test_fused_prenorm_agrees_with_separate_calls(pkg, lib):
    """Same module, same input: `x + m(norm(x))[0]` against `m.forward_prenorm(x, norm)`.  Routing
    can differ on a token whose k-th and (k+1)-th logits are within bf16 rounding of each other,
    so the comparison is norm-wise."""
    for x_dt in (torch.float32, torch.bfloat16):
        cfg, m, norm, x, dy, B, T = _fused_case(pkg, x_dt)
        if x_dt == torch.bfloat16:  # a model converted as a whole, norm weight included
            m, norm = m.to(torch.bfloat16), norm.to(torch.bfloat16)
        ctx = torch.autocast("cuda", dtype=torch.bfloat16, enabled=(x_dt == torch.float32))
        params = list(m.parameters()) + [norm.weight]
        res = []
        for fused in (False, True):
            for p in params:
                p.grad = None
            x.grad = None
            with ctx:
                out = m.forward_prenorm(x, norm)[0] if fused else x + m(norm(x))[0]
            assert out.dtype == x_dt
            out.backward(dy)
            res.append([out.detach().float()] + [x.grad.float()] + [p.grad.float() for p in params])
        for a, b_ in zip(*res):
            rel = ((a - b_).norm() / a.norm().clamp_min(1e-30)).item()
            assert rel < 2e-2, rel
        _say(f"  fused vs separate ({x_dt}): all within 2e-2 norm-wise")


def test_block_with_fused_prenorm(pkg, lib):
    cfg = pkg.ModelConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, num_experts=8,
                          num_experts_per_tok=2, moe_intermediate_size=128, init_std=0.05, use_moe=True)
    a = pkg.Block(cfg, 2)
    b = pkg.Block(cfg, 2, fused_prenorm=True)
    b.load_state_dict(a.state_dict())
    g = torch.Generator().manual_seed(41)
    x = torch.randn(2, 128, 256, generator=g).cuda()
    dy = torch.randn(2, 128, 256, generator=g).cuda()
    outs = []
    for blk in (a, b):
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            o = blk(xi)
        o.backward(dy)
        outs.append((o.detach(), xi.grad, blk.ln_2.weight.grad, blk.attn.c_proj.weight.grad))
    for u, v in zip(*outs):
        rel = ((u - v).norm() / u.norm()).item()
        assert rel < 2e-2, rel


@pytest.mark.parametrize("T,H,I,E,k", [(1, 64, 32, 4, 2), (37, 72, 40, 3, 3), (130, 2048, 64, 16, 4), (300, 520, 264, 6, 1)])
def test_prenorm_moe_odd_shapes(pkg, lib, T, H, I, E, k):
    """`prenorm_moe` (functional entry) against the oracle on shapes off the beaten track, fp32
    residual stream: the MoE oracle on the device's own normalised rows and logits, then the
    norm's autograd on the CPU."""
    _say("prenorm_moe odd shape", T, H, I, E, k)
    g = torch.Generator().manual_seed(7000 + T + H + I + E + k)
    x = (torch.randn(T, H, generator=g) * 1.5)
    nw = 1.0 + 0.2 * torch.randn(H, generator=g)
    bf = lambda *s_, std: (torch.randn(*s_, generator=g) * std).to(torch.bfloat16)
    wr, w1, w3, w2 = bf(E, H, std=0.3), bf(E, I, H, std=0.08), bf(E, I, H, std=0.08), bf(E, H, I, std=0.08)
    dy = torch.randn(T, H, generator=g)
    xd = x.cuda().requires_grad_(True)
    nwd = nw.cuda().requires_grad_(True)
    wd = [w.cuda().requires_grad_(True) for w in (wr, w1, w3, w2)]
    out, logits = pkg.prenorm_moe(xd, nwd, *wd, k, eps=EPS)
    out.backward(dy.cuda())
    xn, _ = pkg.ops.rmsnorm_fwd(xd.detach(), nwd.detach(), EPS)
    lg = logits.detach().cpu()
    f = O.moe_forward(xn.cpu(), wr, w1, w3, w2, k, logits=lg)
    b = O.moe_backward(f, dy, wr, w1, w3, w2)
    fe = O.moe_forward(xn.cpu(), wr, w1, w3, w2, k, logits=lg, emulate_bf16=True)
    be = O.moe_backward(fe, dy, wr, w1, w3, w2, emulate_bf16=True)
    check("out", out, x + f["out"], say=_say)
    for key, t in (("dw1", wd[1].grad), ("dw3", wd[2].grad), ("dw2", wd[3].grad), ("dwr", wd[0].grad)):
        if key == "dwr" and T < 4:  # ill-conditioned difference of gate gradients: see test_gpu_layer
            check(key + " (vs the bf16-rounding oracle)", t, be[key], say=_say)
        else:
            check(key, t, b[key], be[key], say=_say)
    def through_norm(dxn):
        xa = x.clone().requires_grad_(True)
        wa = nw.clone().requires_grad_(True)
        BO.rmsnorm(xa, wa, EPS).backward(dxn)
        return dy + xa.grad, wa.grad
    dx_ref, dnw_ref = through_norm(b["dx"])
    dx_e, dnw_e = through_norm(be["dx"])
    if T < 4:
        check("dx (vs the bf16-rounding oracle)", xd.grad, dx_e, say=_say)
        check("d norm weight (vs the bf16-rounding oracle)", nwd.grad, dnw_e, say=_say)
    else:
        check("dx", xd.grad, dx_ref, dx_e, say=_say)
        check("d norm weight", nwd.grad, dnw_ref, dnw_e, say=_say)


def _random_norm_router_shapes(n, seed):
    import numpy as np
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        E = int(rng.integers(1, 9)) * 16
        out.append((int(rng.integers(1, 600)), int(rng.integers(1, 129)) * 32, E, int(rng.integers(1, min(E, 64) + 1)),
                    torch.float32 if rng.random() < 0.5 else torch.bfloat16))
    return out


@pytest.mark.parametrize("T,H,E,k,x_dt", [
    (1, 64, 16, 2, torch.float32), (37, 256, 32, 4, torch.float32), (300, 1024, 64, 8, torch.bfloat16),
    (8192, 2048, 64, 8, torch.float32), (130, 4096, 128, 64, torch.bfloat16), (17, 2048, 48, 3, torch.float32),
] + _random_norm_router_shapes(8, 5150))
def test_norm_router_topk_in_one_kernel(pkg, lib, T, H, E, k, x_dt):
    """RMSNorm + router product + top-k in one kernel against the three separate steps: xn and
    rstd are the same bits as the norm kernel's; the logits equal the library product on those
    rows to bf16 rounding (another summation order); ids and gates are exactly what the router
    kernel selects on the logits this kernel returned, and exactly the oracle's selection."""
    ops = pkg.ops
    _say(f"norm + router + top-k fused: T={T} H={H} E={E} k={k} x {x_dt}")
    assert ops.rmsnorm_router_supported(H, E, k)
    g = torch.Generator().manual_seed(900 + T + H + E)
    x = (torch.randn(T, H, generator=g) * 1.4).to(x_dt).cuda()
    w = (1.0 + 0.2 * torch.randn(H, generator=g)).cuda()
    wr = (torch.randn(E, H, generator=g) * 0.05).to(torch.bfloat16).cuda()
    xn0, rstd0 = ops.rmsnorm_fwd(x, w, EPS)
    xn, rstd, logits, ids, gates = ops.rmsnorm_router_fwd(x, w, EPS, wr, k)
    assert torch.equal(xn, xn0) and torch.equal(rstd, rstd0)
    assert logits.dtype == torch.bfloat16 and logits.shape == (T, E)
    want = xn.float() @ wr.float().t()
    check("logits", logits, want.cpu(), say=_say)
    # never further from the fp32 product than bf16 rounding plus fp32 summation-order noise
    assert ((logits.float() - want).abs() <= want.abs() * 2.0 ** -8 + 1e-3).all()
    ids2, gates2 = ops.router_topk(logits, k, None)
    assert torch.equal(ids, ids2) and torch.equal(gates, gates2)
    oid, sel = O.topk_select(logits.cpu(), k)
    assert torch.equal(ids.cpu().reshape(T, k), torch.from_numpy(oid).to(torch.int32))
    assert torch.allclose(gates.cpu().reshape(T, k), O.gates_from_selected(sel), atol=1e-6, rtol=1e-5)
    again = ops.rmsnorm_router_fwd(x, w, EPS, wr, k)
    assert all(torch.equal(a, b) for a, b in zip(again, (xn, rstd, logits, ids, gates)))  # reproducible


def test_norm_router_unsupported_shapes_fall_back(pkg, lib):
    ops = pkg.ops
    assert not ops.rmsnorm_router_supported(8192, 64, 8)      # rows too long for the block's LDS tile
    assert not ops.rmsnorm_router_supported(2048, 24, 2)      # experts not a multiple of 16
    assert not ops.rmsnorm_router_supported(2048, 256, 8)
    assert not ops.rmsnorm_router_supported(72, 16, 2)        # rows not a multiple of the 32-wide k-step
    with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_LIMIT"):
        ops.rmsnorm_router_fwd(torch.zeros(4, 72, device="cuda"), torch.ones(72, device="cuda"), EPS,
                               torch.zeros(16, 72, dtype=torch.bfloat16, device="cuda"), 2)
    # prenorm_moe on such a shape takes the separate kernels and still matches (covered by
    # test_prenorm_moe_odd_shapes: H = 72 and 520, E = 3 and 6)
