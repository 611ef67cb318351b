"""`torch.compile` over the MoE module (the reference's `--use_compile`, training/trainer.py:130-131):
the layer body is a pair of registered operators, so the tracer keeps the whole forward in
one graph (`fullgraph=True` raises on any break) and differentiates through it.  Compiled and
eager calls run the same kernels on the same bits, so everything must be bit-identical but the
router weight gradient (a library product in the traced route, the split-k kernel in the eager
one) and, with bf16 tensors, the input gradient (rounded once in the eager call, twice in the
traced one)."""
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_compiled_module_is_one_graph_and_matches_eager(pkg, lib, dtype):
    _say("torch.compile(MoE, fullgraph=True), parameters", dtype)
    m, x, dy = _case(pkg, dtype)
    ctx = lambda: torch.autocast("cuda", dtype=torch.bfloat16, enabled=(dtype == torch.float32))

    def run(mod):
        m.zero_grad(set_to_none=True)
        xi = x.clone().requires_grad_(True)
        with ctx():
            out, logits = mod(xi)
        out.backward(dy)
        return [out.detach(), logits.detach(), xi.grad] + [p.grad.clone() for p in m.parameters()]

    eager = run(m)
    compiled = run(torch.compile(m, backend="aot_eager", fullgraph=True))
    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    for n, a, b in zip(names, eager, compiled):
        assert a.dtype == b.dtype and a.shape == b.shape, n
        if n == "router.weight" or (n == "dx" and dtype == torch.bfloat16):
            # router.weight: library product vs split-k kernel.  dx in bf16: the eager call sums
            # the expert and router contributions in fp32 inside one kernel and rounds once, the
            # traced route rounds each to bf16 and lets autograd add them
            rel = ((a.float() - b.float()).norm() / a.float().norm()).item()
            assert rel < 1e-2, (n, rel)
        else:
            assert torch.equal(a, b), n
    # inference: nothing saved, no gradient
    with torch.no_grad(), ctx():
        o2, _ = torch.compile(m, backend="aot_eager", fullgraph=True)(x)
    assert torch.equal(o2, eager[0])


def test_compiled_with_the_inductor_backend(pkg, lib):
    """The default backend of `torch.compile` (inductor: its generated kernels surround the
    registered operators): one graph, results norm-wise equal to eager (the code around the layer
    is regenerated, so bits may differ), expert kernels bit-equal given equal logits."""
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
    same_logits = torch.equal(eager[1], compiled[1])
    for n, a, b in zip(names, eager, compiled):
        assert a.dtype == b.dtype and a.shape == b.shape, n
        rel = ((a.float() - b.float()).norm() / a.float().norm().clamp_min(1e-30)).item()
        _say(f"  {n}: rel {rel:.2e}")
        assert rel < 1e-2, (n, rel)
        if same_logits and n in ("out", "experts_gate_weights", "experts_up_weights", "experts_down_weights"):
            assert torch.equal(a, b), n


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
