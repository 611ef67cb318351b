"""CPU-side checks: the C ABI library loads and exports every symbol the header declares,
the Python binding mirrors the header, and the module's constructor contract holds.
No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT, load_pkg


def _header_functions():
    text = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", text)


def _ensure_built(pkg):
    if not os.path.exists(pkg.lib.LIB_PATH):
        pkg.build.build_library()


def test_library_exports_every_declared_symbol():
    pkg = load_pkg()
    from importlib import import_module
    pkg.build = import_module(pkg.__name__ + ".build")
    _ensure_built(pkg)
    names = _header_functions()
    assert len(names) >= 15
    cdll = ctypes.CDLL(pkg.lib.LIB_PATH)
    for n in names:
        assert hasattr(cdll, n), n
    assert sorted(names) == sorted(pkg.lib.SIGNATURES)
    L = pkg.lib.load()
    assert L.abi_version == 100
    assert L.cdll.moe_dispatch_workspace_bytes(1000, 8) == 4 * (8 + 1) * 4


def test_module_constructor_contract_cpu():
    pkg = load_pkg()
    cfg = pkg.ModelConfig(hidden_size=64, num_experts=4, num_experts_per_tok=2, moe_intermediate_size=32)
    m = pkg.MoE(cfg)
    assert m.top_k == 2 and m.num_local_experts == 4 and m.ep_size == 1
    sd = m.state_dict()
    assert {k: tuple(v.shape) for k, v in sd.items()} == {
        "router.weight": (4, 64), "experts_gate_weights": (4, 32, 64),
        "experts_up_weights": (4, 32, 64), "experts_down_weights": (4, 64, 32)}
    assert all(v.dtype == torch.float32 for v in sd.values())
    assert pkg.MoE(cfg, 3).top_k == 3
    with pytest.raises(AssertionError):
        pkg.MoE(cfg, 5)
    for attr in ("device", "config", "num_experts", "hidden_size", "intermediate_size",
                 "grouped_gemm_supported", "router", "experts_act_fn"):
        assert hasattr(m, attr)
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="GPU"):
            m(torch.zeros(1, 2, 64))


def test_synthetic_configs_are_seeded_and_shaped():
    pkg = load_pkg()
    a = pkg.configs.make_inputs(1)
    b = pkg.configs.make_inputs(1)
    assert all(torch.equal(a[k], b[k]) for k in ("x", "wr", "w1", "w3", "w2"))
    assert a["x"].shape == (2048, 1024) and a["w1"].shape == (8, 512, 1024) and a["w2"].shape == (8, 1024, 512)
    c4 = pkg.configs.make_inputs(4, scale_tokens=1 / 16)
    counts = torch.bincount(c4["ids"], minlength=16)
    assert (counts == 0).sum() >= 2 and counts.sum() == c4["x"].shape[0]
    assert pkg.configs.gemm_flops(pkg.configs.SHAPES[3]) == 4947802324992


def test_registered_operators_propagate_shapes_without_a_gpu():
    """The fake (shape and dtype only) implementations of the layer's registered operators,
    which are what `torch.compile` traces with: exercised under FakeTensorMode, no kernel runs."""
    import importlib

    import torch
    from torch._subclasses.fake_tensor import FakeTensorMode

    from conftest import PKG_NAME
    traced = importlib.import_module(PKG_NAME + ".traced")
    T, H, E, I, k = 48, 128, 8, 32, 2
    bf, f32, i32 = torch.bfloat16, torch.float32, torch.int32
    with FakeTensorMode():
        for wdt in (f32, bf):
            x = torch.empty(T, H, device="cuda", dtype=f32)
            lg = torch.empty(T, E, device="cuda", dtype=bf)
            ws = [torch.empty(E, I, H, device="cuda", dtype=wdt), torch.empty(E, I, H, device="cuda", dtype=wdt),
                  torch.empty(E, H, I, device="cuda", dtype=wdt)]
            for train in (True, False):
                o = traced.ffn_fwd(x, lg, *ws, k, train)
                shapes = [tuple(t.shape) for t in o]
                gu = (T * k, I) if train else (0,)
                cp = [tuple(w.shape) if wdt == f32 else (0,) for w in ws]
                assert shapes == [(T, H), (T * k,), (T * k,), (E + 1,), (T * k,), (T * k,), (T * k, H), gu, gu,
                                  (T * k, I)] + cp
                assert [t.dtype for t in o[:6]] == [f32, i32, f32, i32, i32, i32]
                assert all(t.dtype == bf for t in o[6:])
            out, ids, gates, offs, p2r, r2p, xp, g, u, act, w1b, w3b, w2b = traced.ffn_fwd(x, lg, *ws, k, True)
            wb = ws if wdt == bf else [w1b, w3b, w2b]
            d = traced.ffn_bwd(out, xp, g, u, act, gates, ids, offs, p2r, r2p, *wb, k, True, False, wdt == f32)
            assert [tuple(t.shape) for t in d] == [(T, H), (T, E)] + [tuple(w.shape) for w in ws]
            assert [t.dtype for t in d] == [f32, bf, wdt, wdt, wdt]
