"""The MoE module inside a GPT-MoE block (benchmark configuration 5, reduced size): fp32
parameters and residual stream, bf16 autocast, forward and backward.

The attention half is stock torch and is only checked loosely against the CPU block oracle
(bf16 autocast vs fp32).  The MoE half is checked to the usual bar on exactly the input and
router logits it received inside the block, captured with hooks."""
import pytest
import torch

from oracle import block_oracle as BO
from oracle import moe_oracle as O
from _tol import check

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


def test_block_forward_backward(pkg, lib):
    assert torch.cuda.is_available()
    cfg = pkg.ModelConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, num_experts=8,
                          num_experts_per_tok=2, moe_intermediate_size=128, init_std=0.05, use_moe=True)
    blk = pkg.Block(cfg, 2)
    B, T, H = 2, 128, 256
    g = torch.Generator().manual_seed(21)
    x = torch.randn(B, T, H, generator=g).cuda().requires_grad_(True)
    dy = torch.randn(B, T, H, generator=g).cuda()
    seen = {}
    blk.mlp.register_forward_hook(lambda m, inp, out: seen.update(moe_in=inp[0].detach(), moe_out=out[0].detach(),
                                                                   logits=out[1].detach()))
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out = blk(x)
    assert out.dtype == torch.float32 and out.shape == (B, T, H)
    out.backward(dy)
    torch.cuda.synchronize()
    for n, p_ in blk.named_parameters():
        assert p_.grad is not None and torch.isfinite(p_.grad).all(), n
    assert torch.isfinite(x.grad).all()

    r = lambda t: t.detach().cpu().to(torch.bfloat16).float()  # what autocast feeds the GEMMs
    P = {"ln1": blk.ln_1.weight.detach().cpu(), "ln2": blk.ln_2.weight.detach().cpu(),
         "wq": r(blk.attn.q_proj.weight), "wk": r(blk.attn.k_proj.weight), "wv": r(blk.attn.v_proj.weight),
         "wc": r(blk.attn.c_proj.weight), "wr": r(blk.mlp.router.weight), "w1": r(blk.mlp.experts_gate_weights),
         "w3": r(blk.mlp.experts_up_weights), "w2": r(blk.mlp.experts_down_weights)}
    ref_out, aux = BO.block_forward(x.detach().cpu(), P, 4, 2, 2)
    # attention half, loose: everything up to the MoE input
    d = (seen["moe_in"].float().cpu() - aux["moe_in"])
    rel = (d.norm() / aux["moe_in"].norm()).item()
    _say(f"  MoE input (after attention + ln_2): rel_fro {rel:.3e}")
    assert rel < 3e-2
    # MoE half, to the usual bar, on the very input and logits the module saw
    m_in = seen["moe_in"].reshape(B * T, H).cpu().to(torch.bfloat16)
    f = O.moe_forward(m_in, P["wr"], P["w1"], P["w3"], P["w2"], 2, logits=seen["logits"].reshape(B * T, 8).cpu())
    check("moe_out in block", seen["moe_out"].reshape(B * T, H), f["out"], say=_say)
    # and the whole block against the oracle, loosely
    rel = ((out.detach().cpu() - ref_out).norm() / ref_out.norm()).item()
    _say(f"  block output: rel_fro {rel:.3e}")
    assert rel < 3e-2


def test_config5_real_shape_moe_inside_block(pkg, lib):
    """Benchmark configuration 5 at its real shape (hidden 2048, 32 query / 8 KV heads of 64,
    seq 4096 x batch 2, 64 experts top-8, FFN 1024; fp32 parameters, bf16 autocast): the MoE
    inside the block against the MoE oracle on exactly the rows and router logits it received,
    forward and backward, first with the caller's three separate calls (model/gpt.py:32-33), then
    with the norm and the residual add inside the layer's call."""
    assert torch.cuda.is_available()
    s = pkg.configs.SHAPES[5]
    B, T, H, E, k = 2, 4096, s.H, s.E, s.k
    cfg = pkg.ModelConfig(hidden_size=H, num_attention_heads=32, num_key_value_heads=8, num_experts=E,
                          num_experts_per_tok=k, moe_intermediate_size=s.I, init_std=0.02, use_moe=True,
                          seed=pkg.configs.BASE_SEED, vocab_size=50304)
    blk = pkg.Block(cfg, k)
    wte = torch.nn.Embedding(cfg.vocab_size, H, device="cuda")
    torch.nn.init.normal_(wte.weight, mean=0.0, std=0.02)
    g = torch.Generator().manual_seed(pkg.configs.BASE_SEED)
    ids = torch.randint(0, cfg.vocab_size, (B, T), generator=g).cuda()
    dy = torch.randn(B, T, H, generator=g)
    dyd = dy.cuda()
    names = ("experts_gate_weights", "experts_up_weights", "experts_down_weights")
    r = lambda t: t.detach().cpu().to(torch.bfloat16)  # what autocast / the cast kernel feed the GEMMs
    wr, w1, w3, w2 = r(blk.mlp.router.weight), *[r(getattr(blk.mlp, n)) for n in names]
    dy2 = dy.reshape(B * T, H)

    def oracle_checks(tag, rows_bf16, logits, moe_out, base=None):
        lg = logits.reshape(B * T, E).cpu()
        f = O.moe_forward(rows_bf16, wr, w1, w3, w2, k, logits=lg)
        b = O.moe_backward(f, dy2, wr, w1, w3, w2)
        fe = O.moe_forward(rows_bf16, wr, w1, w3, w2, k, logits=lg, emulate_bf16=True)
        be = O.moe_backward(fe, dy2, wr, w1, w3, w2, emulate_bf16=True)
        ref_out = f["out"] if base is None else base + f["out"]
        check(f"{tag} out", moe_out.reshape(B * T, H), ref_out, say=_say)
        for n, key in zip(names + ("router.weight",), ("dw1", "dw3", "dw2", "dwr")):
            p = blk.mlp.router.weight if key == "dwr" else getattr(blk.mlp, n)
            assert p.grad is not None and p.grad.dtype == torch.float32
            check(f"{tag} {key}", p.grad, b[key], be[key], say=_say)
        return f, b, be

    # ---- the caller's three separate calls
    seen = {}

    def spy(mod, inp, out):
        seen.update(moe_in=inp[0].detach(), moe_out=out[0].detach(), logits=out[1].detach())
        inp[0].register_hook(lambda gr: seen.update(d_moe_in=gr.detach()))

    hook = blk.mlp.register_forward_hook(spy)
    _say("config 5 real shape: separate norm / layer / residual add")
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out_a = blk(wte(ids))
    assert out_a.dtype == torch.float32 and out_a.shape == (B, T, H)
    out_a.backward(dyd)
    hook.remove()
    assert seen["moe_out"].dtype == torch.float32 and seen["logits"].dtype == torch.bfloat16
    f, b, be = oracle_checks("separate:", r(seen["moe_in"]).reshape(B * T, H), seen["logits"], seen["moe_out"])
    check("separate: d moe_in", seen["d_moe_in"].reshape(B * T, H), b["dx"], be["dx"], say=_say)
    grads_a = [p.grad.clone() for p in blk.parameters()] + [wte.weight.grad.clone()]
    del f, b, be

    # ---- norm and residual add inside the layer's call
    _say("config 5 real shape: ln_2 and the residual add inside the layer's call")
    blk.zero_grad(set_to_none=True)
    wte.zero_grad(set_to_none=True)
    blk.fused_prenorm = True
    inner = blk.mlp.forward_prenorm

    def spy2(x, norm, add_residual=True):
        res = inner(x, norm, add_residual)
        seen.update(h=x.detach(), fused_out=res[0].detach(), fused_logits=res[1].detach())
        return res

    blk.mlp.forward_prenorm = spy2
    with torch.autocast("cuda", dtype=torch.bfloat16):
        out_b = blk(wte(ids))
    out_b.backward(dyd)
    del blk.mlp.forward_prenorm
    h2 = seen["h"].reshape(B * T, H)
    xn, _ = pkg.ops.rmsnorm_fwd(h2, blk.ln_2.weight.detach(), blk.ln_2.variance_epsilon)  # same bits again
    oracle_checks("fused:", xn.cpu(), seen["fused_logits"], seen["fused_out"], base=h2.cpu())
    # the two ways of calling agree (routing may differ on tokens with near-tied logits: norm-wise)
    grads_b = [p.grad for p in blk.parameters()] + [wte.weight.grad]
    for u, v in zip([out_a.detach()] + grads_a, [out_b.detach()] + grads_b):
        rel = ((u - v).norm() / u.norm().clamp_min(1e-30)).item()
        assert rel < 2e-2, rel


@pytest.mark.parametrize("fused", [False, True])
def test_block_under_deterministic_algorithms(pkg, lib, fused):
    """The trainer's `--deterministic` switch (utils/training.py:82,
    `torch.use_deterministic_algorithms(True)`): nothing in the layer's path raises under it
    (torch then also fills every `torch.empty` with NaN, so a kernel that left part of an output
    unwritten would show), and two steps give the same bits."""
    torch.use_deterministic_algorithms(True)
    try:
        cfg = pkg.ModelConfig(hidden_size=256, num_attention_heads=4, num_key_value_heads=2, num_experts=8,
                              num_experts_per_tok=2, moe_intermediate_size=256, init_std=0.05, use_moe=True)
        blk = pkg.Block(cfg, 2, fused_prenorm=fused)
        g = torch.Generator().manual_seed(5)
        x = torch.randn(2, 128, 256, generator=g).cuda().requires_grad_(True)
        dy = torch.randn(2, 128, 256, generator=g).cuda()
        runs = []
        for _ in range(2):
            blk.zero_grad(set_to_none=True)
            x.grad = None
            with torch.autocast("cuda", dtype=torch.bfloat16):
                out = blk(x)
            out.backward(dy)
            runs.append([out.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in blk.parameters()])
        assert all(torch.isfinite(t).all() for t in runs[0])
        assert all(torch.equal(a, b) for a, b in zip(*runs))
    finally:
        torch.use_deterministic_algorithms(False)
