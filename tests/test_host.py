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
    assert L.abi_version == 101
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
                gu = (traced.gu_blocked_bytes(T * k, E, I),) if train else (0,)
                cp = [tuple(w.shape) if wdt == f32 else (0,) for w in ws]
                assert shapes == [(T, H), (T * k,), (T * k,), (E + 1,), (T * k,), (T * k,), (T * k, H), gu,
                                  (T * k, I)] + cp
                assert [t.dtype for t in o[:6]] == [f32, i32, f32, i32, i32, i32]
                assert o[7].dtype == torch.uint8 and all(t.dtype == bf for t in o[6:7] + o[8:])
            out, ids, gates, offs, p2r, r2p, xp, gu, act, w1b, w3b, w2b = traced.ffn_fwd(x, lg, *ws, k, True)
            wb = ws if wdt == bf else [w1b, w3b, w2b]
            d = traced.ffn_bwd(out, xp, gu, act, gates, ids, offs, p2r, r2p, *wb, k, True, False, wdt == f32)
            assert [tuple(t.shape) for t in d] == [(T, H), (T, E)] + [tuple(w.shape) for w in ws]
            assert [t.dtype for t in d] == [f32, bf, wdt, wdt, wdt]
            # the pair with the router product inside: bf16 copies only of what is not bf16 already
            for xdt in (f32, bf):
                xr = torch.empty(T, H, device="cuda", dtype=xdt)
                wr = torch.empty(E, H, device="cuda", dtype=wdt)
                for train in (True, False):
                    o = traced.routed_fwd(xr, wr, *ws, k, train)
                    R = T * k
                    kept = lambda shape, made: tuple(shape) if (train and made) else (0,)
                    assert [tuple(t.shape) for t in o] == [
                        (T, H), (T, E), (R,), (R,), (E + 1,), (R,), (R,), kept((T, H), xdt == f32),
                        kept((E, H), wdt == f32), kept((R, H), True),
                        (traced.gu_blocked_bytes(R, E, I) if train else 0,), kept((R, I), True)] + [
                        tuple(w.shape) if wdt == f32 else (0,) for w in ws]
                    assert [t.dtype for t in o[:7]] == [xdt, bf, i32, f32, i32, i32, i32]
                    assert o[10].dtype == torch.uint8 and all(t.dtype == bf for t in o[7:10] + o[11:])
                (out, logits, ids, gates, offs, p2r, r2p, xn, wrb, xp, gu, act, w1b, w3b, w2b) = traced.routed_fwd(
                    xr, wr, *ws, k, True)
                wb = ws if wdt == bf else [w1b, w3b, w2b]
                for ext in (None, logits):
                    d = traced.routed_bwd(out, ext, xr if xdt == bf else xn, wr if wdt == bf else wrb, xp, gu, act,
                                          gates, ids, offs, p2r, r2p, *wb, k, xdt == f32, wdt == f32, wdt == f32)
                    assert [tuple(t.shape) for t in d] == [(T, H), (E, H)] + [tuple(w.shape) for w in ws]
                    assert [t.dtype for t in d] == [xdt, wdt, wdt, wdt, wdt]


def test_traced_buffer_size_is_the_library_s(lib):
    """The size the traced forward operator's shape function gives the blocked g/u buffer is the
    one the library reports (and the wrapper allocates), over ragged and empty shapes."""
    import importlib

    from conftest import PKG_NAME
    traced = importlib.import_module(PKG_NAME + ".traced")
    for R in (0, 1, 255, 256, 257, 4096, 131072, 131073):
        for E in (1, 8, 64, 1024):
            for I in (32, 48, 1024, 1056):
                assert traced.gu_blocked_bytes(R, E, I) == max(lib.cdll.moe_gu_blocked_bytes(R, E, I), 16)


def test_mfu_table_for_amd_parts(monkeypatch):
    """`profile.py` mirrors utils/profile.py:3-48 for AMD Instinct parts: same function names,
    arguments and return values, so the reference's MFU line works on an MI355X."""
    pkg = load_pkg()
    prof = pkg.profile
    assert prof.peak_for_device_name("AMD Instinct MI355X", "bf16") == 2.5e15
    assert prof.peak_for_device_name("AMD Instinct MI355X", "FP8") == 5.0e15
    assert prof.peak_for_device_name("AMD Instinct MI300X", "bf16") == 1307.4e12
    assert prof.peak_for_device_name("NVIDIA H100", "bf16") == 0.0
    assert set(prof.GPU_PEAK_FLOPS["MI355X"]) >= {"fp32", "fp16", "bf16"}   # the reference's keys
    monkeypatch.setattr(torch.cuda, "get_device_name", lambda i=0: "AMD Instinct MI355X")
    monkeypatch.setattr(torch.cuda, "device_count", lambda: 8)
    assert prof.get_gpu_peak_flops("bf16") == 2.5e15
    assert prof.get_gpu_peak_flops("bf16", per_device=False) == 8 * 2.5e15

    class Model:
        def get_flops_per_fwd_bwd(self, batch_size, seq_len):
            return 1.0e15 * batch_size

    mfu, achieved, peak = prof.compute_mfu(Model(), batch_size=2, seq_len=4096, time=2.0, ga=4)
    assert peak == 2.5e15 and achieved == 4.0e15 and abs(mfu - 1.6) < 1e-12
    assert prof.compute_mfu(Model(), 1, 1, 0.0)[0] == 0


def test_launch_observer_sees_every_entry_point_call():
    """`MoELib.observer` is called around every entry point (bench.py hangs HIP events on it).
    A null pointer is refused by the argument checks before anything touches a GPU, so this
    runs on the CPU."""
    pkg = load_pkg()
    L = pkg.lib.load()
    seen = []

    class Obs:
        def before(self, name):
            seen.append(("before", name))

        def after(self, name):
            seen.append(("after", name))

    L.observer = Obs()
    try:
        with pytest.raises(pkg.lib.MoELibError, match="MOE_ERR_NULL"):
            L.call("moe_cast_f32_bf16", None, None, 8, None)
        L.call("moe_cast_f32_bf16", None, None, 0, None)  # nothing to do: returns 0
    finally:
        L.observer = None
    assert seen == [("before", "moe_cast_f32_bf16"), ("after", "moe_cast_f32_bf16")] * 2
    L.call("moe_cast_f32_bf16", None, None, 0, None)
    assert len(seen) == 4


# pointers an entry point may be handed as null (documented so in the header); every other
# pointer must be refused with MOE_ERR_NULL before anything is launched
_OPTIONAL_POINTERS = {
    "moe_router_topk_fwd": {"bias"},
    "moe_histogram_scan_checked": {"bad_ids"}, "moe_histogram_scan_static": {"bad_ids"},
    "moe_permute_bwd": {"addend"},
    "moe_gemm_dgrad_down_swiglu_bwd_packed": {"dgate_part"},
    "moe_gemm_dgrad_down_swiglu_bwd_blocked": {"dgate_part"},
    "moe_combine_fwd": {"gates"}, "moe_combine_fwd_residual": {"gates"},
    "moe_combine_bwd": {"gates"}, "moe_combine_bwd_by_token": {"gates"},
    "moe_rmsnorm_bwd": {"d2", "dres"},
    "moe_ffn_forward": {"bias"},
    "moe_f32_combine_fwd": {"gates"}, "moe_f32_combine_bwd": {"y", "gates", "dgates"},
}


def test_every_required_pointer_is_checked_before_any_launch():
    """Each entry point, with each of its required pointers null in turn (the others point at
    host memory, sizes are small and valid): MOE_ERR_NULL comes back, i.e. the argument checks
    stop the call before a kernel could see the pointer.  Nothing is launched, so this runs
    without a GPU (and is harmless with one)."""
    pkg = load_pkg()
    L = pkg.lib.load()
    text = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    host = ctypes.create_string_buffer(1 << 20)
    base = (ctypes.addressof(host) + 255) & ~255
    sizes = {"T": 8, "E": 16, "k": 2, "H": 64, "I": 256, "R": 16, "M": 64, "N": 64, "S": 2, "P": 1, "n": 64}
    checked = 0
    for name, (res, args) in pkg.lib.SIGNATURES.items():
        if res is not ctypes.c_int or ctypes.c_void_p not in args:
            continue
        params = re.search(r"\b" + name + r"\s*\(([^)]*)\)", text).group(1).replace("\n", " ").split(",")
        pnames = [re.split(r"[\s\*]+", p.strip())[-1] for p in params]
        assert len(pnames) == len(args), name
        optional = _OPTIONAL_POINTERS.get(name, set()) | {"stream"}
        for null_at, (a, n) in enumerate(zip(args, pnames)):
            if a is not ctypes.c_void_p or n in optional:
                continue
            vals = []
            for i, (b, m) in enumerate(zip(args, pnames)):
                if b is ctypes.c_void_p:
                    vals.append(None if (i == null_at or m == "stream") else base + 4096 * i)
                elif b is ctypes.c_int64:
                    vals.append(sizes.get(m, (1 << 20) if "bytes" in m else 8))
                elif b is ctypes.c_float:
                    vals.append(1e-6)
                else:
                    vals.append(0)
            rc = getattr(L.cdll, name)(*vals)
            assert rc == -1, f"{name}: null `{n}` gave {rc}, not MOE_ERR_NULL"
            checked += 1
    assert checked > 90


def test_sizes_and_dtypes_are_checked_before_any_launch():
    """Each entry point with each size argument negative and beyond every limit (2^40) in turn,
    and each dtype code invalid: a negative MOE_ERR_* comes back.  Pointers point at host memory,
    so this is for a machine without a GPU only (there a check that let a value through could do
    no harm: the launch itself fails with 'no device')."""
    if torch.cuda.is_available():
        pytest.skip("hands host pointers to the entry points: CPU-only check")
    pkg = load_pkg()
    L = pkg.lib.load()
    text = open(os.path.join(ROOT, "include", "moe_gfx950.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    host = ctypes.create_string_buffer(1 << 20)
    base = (ctypes.addressof(host) + 255) & ~255
    sizes = {"T": 8, "E": 16, "k": 2, "H": 64, "I": 256, "R": 16, "M": 64, "N": 64, "S": 2, "P": 1, "n": 64}
    # sizes that have no upper limit by design: a byte count the caller vouches for, an element count
    unlimited = {"workspace_bytes", "n"}
    checked = 0
    for name, (res, args) in pkg.lib.SIGNATURES.items():
        if res is not ctypes.c_int or ctypes.c_void_p not in args:
            continue
        params = re.search(r"\b" + name + r"\s*\(([^)]*)\)", text).group(1).replace("\n", " ").split(",")
        pnames = [re.split(r"[\s\*]+", p.strip())[-1] for p in params]

        def call(bad_at, bad):
            vals = []
            for i, (b, m) in enumerate(zip(args, pnames)):
                if b is ctypes.c_void_p:
                    vals.append(None if m == "stream" else base + 4096 * i)
                elif i == bad_at:
                    vals.append(bad)
                elif b is ctypes.c_int64:
                    vals.append(sizes.get(m, (1 << 20) if "bytes" in m else 8))
                elif b is ctypes.c_float:
                    vals.append(1e-6)
                else:
                    vals.append(0)
            return getattr(L.cdll, name)(*vals)

        for i, (a, n) in enumerate(zip(args, pnames)):
            if a is ctypes.c_int64:
                assert call(i, -1) < 0, f"{name}: {n} = -1 accepted"
                if n not in unlimited:
                    assert call(i, (1 << 40) + 8) < 0, f"{name}: {n} = 2^40 + 8 accepted"
                checked += 1
            elif a is ctypes.c_int and "dtype" in n:
                assert call(i, 7) == -4, f"{name}: dtype code 7 for {n} not refused as MOE_ERR_DTYPE"
                checked += 1
    assert checked > 100


def test_precision_rule_of_the_module_cpu():
    """Which calls the module runs in fp32 from end to end: those the reference would (fp32 input,
    fp32 parameters, no autocast), unless the caller asks for the bf16 cores."""
    pkg = load_pkg()
    cfg = pkg.ModelConfig(hidden_size=64, num_experts=4, num_experts_per_tok=2, moe_intermediate_size=32)
    m = pkg.MoE(cfg)
    x = torch.zeros(1, 2, 64)
    assert m._runs_in_fp32(x)
    assert not m._runs_in_fp32(x.to(torch.bfloat16))
    m.bf16_compute_for_fp32_calls = True
    assert not m._runs_in_fp32(x)
    m.bf16_compute_for_fp32_calls = False
    mb = pkg.MoE(cfg).to(torch.bfloat16)
    assert not mb._runs_in_fp32(x) and not mb._runs_in_fp32(x.to(torch.bfloat16))
    m.experts_up_weights.data = m.experts_up_weights.data.to(torch.bfloat16)   # mixed parameters
    assert not m._runs_in_fp32(x)
