"""The layer inside an optimizer loop: a few SGD steps of the module on the GPU against the
same steps taken on the CPU with the oracle's forward and hand-written backward."""
import pytest
import torch

from conftest import load_pkg
from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def P():
    pkg = load_pkg()
    pkg.lib.load()
    assert torch.cuda.is_available(), "GPU tests need an MI355X"
    return pkg


@pytest.mark.parametrize("accumulate_into_grad", [False, True])
def test_sgd_steps_follow_the_oracle(P, accumulate_into_grad):
    """fp32 masters, bf16 autocast, mean-square loss, plain SGD (the reference trainer's step,
    training/trainer.py:209-250, without its parallel wrappers): per-step losses and the
    total update of every parameter against a CPU loop that casts the masters to bf16 each
    step, runs the oracle forward on the device's own logits (so that both sides route alike)
    and applies the oracle's gradients.  Also exercises the bf16 weight copies across
    optimizer steps and, in the second variant, two accumulated micro-steps per update."""
    H, I, E, k, T = 64, 32, 4, 2, 192
    steps, lr, micro = 8, 0.5, (2 if accumulate_into_grad else 1)
    cfg = P.ModelConfig(hidden_size=H, num_experts=E, num_experts_per_tok=k, moe_intermediate_size=I, init_std=0.1)
    m = P.MoE(cfg, k)
    m.accumulate_wgrad_into_grad = accumulate_into_grad
    names = ("router.weight", "experts_gate_weights", "experts_up_weights", "experts_down_weights")
    start = {n: p.detach().cpu().clone() for n, p in m.named_parameters()}
    cpu = {n: start[n].clone() for n in names}
    opt = torch.optim.SGD(m.parameters(), lr=lr)
    g = torch.Generator().manual_seed(5)
    xs = [torch.randn(T, H, generator=g) for _ in range(steps * micro)]
    tg = [torch.randn(T, H, generator=g) * 0.1 for _ in range(steps * micro)]
    bf = torch.bfloat16
    for s in range(steps):
        grads = {n: torch.zeros_like(cpu[n]) for n in names}
        loss_dev = loss_cpu = 0.0
        for j in range(micro):
            x, t = xs[s * micro + j], tg[s * micro + j]
            with torch.autocast("cuda", dtype=bf):
                out, logits = m(x.cuda()[None])
            loss = (out[0] - t.cuda()).pow(2).mean() / micro
            loss.backward()
            loss_dev += loss.item()
            wb = {n: cpu[n].to(bf) for n in names}
            f = O.moe_forward(x.to(bf), wb[names[0]], wb[names[1]], wb[names[2]], wb[names[3]], k,
                              logits=logits[0].detach().cpu())
            loss_cpu += ((f["out"].float() - t).pow(2).mean() / micro).item()
            dy = 2.0 * (f["out"].float() - t) / (T * H) / micro
            b = O.moe_backward(f, dy, wb[names[0]], wb[names[1]], wb[names[2]], wb[names[3]])
            for n, key in zip(names, ("dwr", "dw1", "dw3", "dw2")):
                grads[n] += b[key].float()
        opt.step()
        opt.zero_grad(set_to_none=True)
        for n in names:
            cpu[n] -= lr * grads[n]
        _say(f"  step {s}: loss device {loss_dev:.6f} oracle {loss_cpu:.6f}")
        assert abs(loss_dev - loss_cpu) <= 2e-3 * abs(loss_cpu), (s, loss_dev, loss_cpu)
    dev = dict(m.named_parameters())
    for n in names:
        moved_cpu = cpu[n] - start[n]
        moved_dev = dev[n].detach().cpu() - start[n]
        rel = ((moved_dev - moved_cpu).norm() / moved_cpu.norm()).item()
        _say(f"  {n}: |update| {moved_cpu.norm().item():.3e}, device vs oracle {rel:.3e}")
        assert moved_cpu.norm() > 0 and rel <= 1e-2, n
