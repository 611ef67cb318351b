"""The layer inside a HIP graph: small configurations are bound by the host's launch rate (some
thirty launches per forward+backward), which a captured graph removes.  The library allocates
nothing, never synchronises and records no memset nodes; what is checked here is that a captured
forward+backward, replayed several times with eager work and synchronisations in between and
with fresh inputs copied into the static buffers, reproduces the eager results bit for bit on
every replay (the kernels are deterministic)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("split_wgrad", [True, False])
def test_captured_forward_backward_replays_match_eager(pkg, lib, split_wgrad):
    # 8 experts of 128 x 256: few weight-gradient tiles, so the row-split path (and its sums) is
    # inside the graph; 64 experts of 256 x 512: the plain path
    E, H, I, k = (8, 256, 128, 2) if split_wgrad else (64, 512, 256, 4)
    cfg = pkg.ModelConfig(hidden_size=H, num_experts=E, num_experts_per_tok=k, moe_intermediate_size=I,
                          init_std=0.05)
    m = pkg.MoE(cfg, k)
    B, T = 2, 192
    gen = torch.Generator().manual_seed(61)
    inputs = [(torch.randn(B, T, H, generator=gen).cuda(), torch.randn(B, T, H, generator=gen).cuda())
              for _ in range(4)]
    params = list(m.parameters())

    def eager(x, dy):
        for p in params:
            p.grad = None
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, logits = m(xi)
        out.backward(dy)
        return [out.detach().clone(), logits.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in params]

    want = [eager(x, dy) for x, dy in inputs]

    sx = inputs[0][0].clone().requires_grad_(True)
    sdy = inputs[0][1].clone()

    def step():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, logits = m(sx)
        out.backward(sdy)
        return out, logits

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            for p in params:
                p.grad = None
            sx.grad = None
            step()
    torch.cuda.current_stream().wait_stream(side)
    for p in params:
        p.grad = None
    sx.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_out, s_logits = step()
    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    for rep, ((x, dy), ref) in enumerate(list(zip(inputs, want)) + list(zip(inputs[:2], want[:2]))):
        with torch.no_grad():
            sx.copy_(x)
            sdy.copy_(dy)
        graph.replay()
        torch.cuda.synchronize()
        got = [s_out, s_logits, sx.grad] + [p.grad for p in params]
        for n, a, b in zip(names, got, ref):
            assert torch.equal(a, b), (rep, n)
        # eager work of the same kind between replays (other buffers, same kernels)
        eager(*inputs[(rep + 1) % len(inputs)])
        torch.cuda.synchronize()
        _say(f"  replay {rep}: identical to eager")
        # eager() replaced the .grad tensors; the graph writes into the ones of capture time
        for p, g in zip(params, got[3:]):
            p.grad = g
    del graph


def test_captured_step_follows_the_master_weights(pkg, lib):
    """fp32 master weights change between replays (an optimizer step outside the graph): the graph
    must round them again on every replay instead of replaying with the bf16 copies the module
    held when it was captured."""
    E, H, I, k = 8, 256, 128, 2
    cfg = pkg.ModelConfig(hidden_size=H, num_experts=E, num_experts_per_tok=k, moe_intermediate_size=I,
                          init_std=0.05)
    m = pkg.MoE(cfg, k)
    gen = torch.Generator().manual_seed(67)
    x = torch.randn(2, 96, H, generator=gen).cuda()
    dy = torch.randn(2, 96, H, generator=gen).cuda()
    params = list(m.parameters())

    def eager():
        for p in params:
            p.grad = None
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, logits = m(xi)
        out.backward(dy)
        return [out.detach().clone(), logits.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in params]

    sx = x.clone().requires_grad_(True)

    def step():
        with torch.autocast("cuda", dtype=torch.bfloat16):
            out, logits = m(sx)
        out.backward(dy)
        return out, logits

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # (leaves fresh bf16 copies in the module's cache)
            for p in params:
                p.grad = None
            sx.grad = None
            step()
    torch.cuda.current_stream().wait_stream(side)
    for p in params:
        p.grad = None
    sx.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_out, s_logits = step()
    names = ["out", "gate_logits", "dx"] + [n for n, _ in m.named_parameters()]
    for rep in range(3):
        if rep:
            with torch.no_grad():  # what an optimizer step does: in-place updates of the masters
                for p in params:
                    p.add_(0.02 * torch.randn(p.shape, generator=gen).cuda())
        graph.replay()
        torch.cuda.synchronize()
        got = [s_out.clone(), s_logits.clone(), sx.grad.clone()] + [p.grad.clone() for p in params]
        held = [p.grad for p in params]
        ref = eager()
        for n, a, b in zip(names, got, ref):
            assert torch.equal(a, b), (rep, n)
        _say(f"  replay {rep} after {'an update of' if rep else 'capturing with'} the masters: identical to eager")
        for p, g in zip(params, held):
            p.grad = g
    del graph
