"""`torch.compile` over the MoE module (the reference's `--use_compile`, training/trainer.py:130-131):
the layer body is a pair of registered operators, so the tracer keeps the whole forward in
one graph (`fullgraph=True` raises on any break) and differentiates through it.  Compiled and
eager calls run the same kernels on the same bits (under bf16 autocast or with bf16 tensors the
router product is inside the operator as well), so everything must be bit-identical."""
import importlib

import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def _case(pkg, dtype):
    cfg = pkg.ModelConfig(hidden_size=256, num_experts=8, num_experts_per_tok=2, moe_intermediate_size=128,
                          init_std=0.05)
    m = pkg.MoE(cfg, 2)
    g = torch.Generator().manual_seed(51)
    x = torch.randn(2, 96, 256, generator=g).cuda()
    dy = torch.randn(2, 96, 256, generator=g).cuda()
    if dtype == torch.bfloat16:
        m, x, dy = m.to(dtype), x.to(dtype), dy.to(dtype)
    return m, x, dy


def test_registered_operators_pass_opcheck(pkg, lib):
    traced = importlib.import_module(pkg.__name__ + ".traced")
    m, x, _ = _case(pkg, torch.float32)
    x2 = x.reshape(-1, 256).requires_grad_(True)
    logits = torch.nn.functional.linear(x2.detach().bfloat16(), m.router.weight.detach().bfloat16()).requires_grad_(True)
    args = (x2, logits, m.experts_gate_weights, m.experts_up_weights, m.experts_down_weights, 2, True)
    torch.library.opcheck(traced.ffn_fwd, args,
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
    outs = traced.ffn_fwd(*[a.detach() if isinstance(a, torch.Tensor) else a for a in args])
    out, ids, gates, offs, p2r, r2p, xp, gu, act, w1b, w3b, w2b = outs
    bargs = (torch.randn_like(out), xp, gu, act, gates, ids, offs, p2r, r2p, w1b, w3b, w2b, 2, True, False, True)
    torch.library.opcheck(traced.ffn_bwd, bargs, test_utils=("test_schema", "test_faketensor"))
    # the pair with the router product inside, fp32 and bf16 tensors (bf16: no copies are returned)
    for dt in (torch.float32, torch.bfloat16):
        xr = x2.detach().to(dt).requires_grad_(True)
        ws = [w.detach().to(dt).requires_grad_(True) for w in (m.router.weight, m.experts_gate_weights,
                                                               m.experts_up_weights, m.experts_down_weights)]
        args = (xr, *ws, 2, True)
        torch.library.opcheck(traced.routed_fwd, args,
                              test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
        (out, logits, ids, gates, offs, p2r, r2p, xn, wrb, xp, gu, act, w1b, w3b, w2b) = traced.routed_fwd(
            *[a.detach() if isinstance(a, torch.Tensor) else a for a in args])
        f32 = dt == torch.float32
        assert (xn.numel() > 0) == f32 and (wrb.numel() > 0) == f32 and (w1b.numel() > 0) == f32
        saved = (xn, wrb, w1b, w3b, w2b) if f32 else tuple(t.detach() for t in (xr, *ws))
        for ext in (None, torch.randn_like(logits)):
            bargs = (torch.randn_like(out), ext, saved[0], saved[1], xp, gu, act, gates, ids, offs, p2r, r2p,
                     *saved[2:], 2, f32, f32, f32)
            torch.library.opcheck(traced.routed_bwd, bargs, test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_module_is_one_graph_and_matches_eager(pkg, lib, dtype):
    _say("torch.compile(MoE, fullgraph=True), parameters", dtype)
    m, x, dy = _case(pkg, dtype)
    ctx = lambda: torch.autocast("cuda", dtype=torch.bfloat16, enabled=(dtype == torch.float32))

    def run(mod, aux=False):
        m.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        with ctx():
            out, logits = mod(xi)
        loss = (out.float() * dy.float()).sum()
        if aux:  # a loss on the returned logits as well (a load-balancing term would be one)
            loss = loss + 0.01 * (logits.float() ** 2).sum()
        loss.backward()
        return [out.detach(), logits.detach(), xi.grad] + [p.grad.clone() for p in m.parameters()]

    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    cm = torch.compile(m, backend="aot_eager", fullgraph=True)
    for aux in (False, True):
        eager = run(m, aux)
        compiled = run(cm, aux)
        for n, a, b in zip(names, eager, compiled):
            assert a.dtype == b.dtype and a.shape == b.shape, n
            assert torch.equal(a, b), (n, aux)
    eager = run(m)
    # inference: nothing saved, no gradient
    with torch.no_grad(), ctx():
        o2, _ = torch.compile(m, backend="aot_eager", fullgraph=True)(x)
    assert torch.equal(o2, eager[0])


def test_compiled_with_the_inductor_backend(pkg, lib):
    """The default backend of `torch.compile` (inductor: its generated code surrounds the
    registered operators): one graph and, the router product being inside the operator, the bits
    of the eager call."""
    _say("torch.compile(MoE, backend=inductor, fullgraph=True)")
    m, x, dy = _case(pkg, torch.float32)

    def run(mod):
        m.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, logits = mod(xi)
        out.backward(dy)
        return [out.detach(), logits.detach(), xi.grad] + [p.grad.clone() for p in m.parameters()]

    eager = run(m)
    compiled = run(torch.compile(m, backend="inductor", fullgraph=True))
    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    for n, a, b in zip(names, eager, compiled):
        assert a.dtype == b.dtype and a.shape == b.shape, n
        assert torch.equal(a, b), n


def test_compiled_module_on_the_bf16_cores_for_fp32_calls(pkg, lib):
    """fp32 parameters and input without autocast and `bf16_compute_for_fp32_calls`: the router
    product is then the module's fp32 `nn.Linear` inside the graph and the experts are the
    `ffn_fwd` / `ffn_bwd` pair.  Bits of the eager call, except the router weight gradient (a
    library product here, the split-k kernel there) and its rounding into dx."""
    m, x, dy = _case(pkg, torch.float32)
    m.bf16_compute_for_fp32_calls = True

    def run(mod):
        m.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        out, logits = mod(xi)
        out.backward(dy)
        return [out.detach(), logits.detach(), xi.grad] + [p.grad.clone() for p in m.parameters()]

    eager = run(m)
    compiled = run(torch.compile(m, backend="aot_eager", fullgraph=True))
    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    for n, a, b in zip(names, eager, compiled):
        assert a.dtype == b.dtype and a.shape == b.shape, n
        if n in ("router.weight", "dx", "gate_logits"):
            rel = ((a.float() - b.float()).norm() / a.float().norm()).item()
            assert rel < 1e-2, (n, rel)
        else:
            assert torch.equal(a, b) or not torch.equal(eager[1], compiled[1]), n


def test_compiled_fp32_call_takes_the_fp32_operators(pkg, lib):
    """fp32 parameters and input, no autocast: the compiled module stays one graph, runs the
    fp32 pair of operators and gives the bits of the eager fp32 call (same kernels, same order;
    the router product is the module's own nn.Linear in both)."""
    traced = importlib.import_module(pkg.__name__ + ".traced")
    m, x, dy = _case(pkg, torch.float32)
    x2 = x.reshape(-1, 256).requires_grad_(True)
    logits = torch.nn.functional.linear(x2.detach(), m.router.weight.detach()).requires_grad_(True)
    args = (x2, logits, m.experts_gate_weights, m.experts_up_weights, m.experts_down_weights, 2, True)
    torch.library.opcheck(traced.ffn_f32_fwd, args,
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))

    def run(mod):
        m.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        out, lg = mod(xi)
        out.backward(dy)
        return [out.detach(), lg.detach(), xi.grad] + [p.grad.clone() for p in m.parameters()]

    eager = run(m)
    compiled = run(torch.compile(m, backend="aot_eager", fullgraph=True))
    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    for n, a, b in zip(names, eager, compiled):
        assert a.dtype == torch.float32 and b.dtype == torch.float32 and a.shape == b.shape, n
        rel = ((a - b).norm() / a.norm().clamp_min(1e-30)).item()
        _say(f"  {n}: rel diff compiled vs eager {rel:.2e}")
        assert rel < 1e-5, (n, rel)
    assert torch.equal(eager[0], compiled[0])
