"""Floating-point acceptance rule shared by the GPU parity tests.

The bar is rtol = atol = 1e-2 against the fp32 oracle on identical bf16 inputs.  Tensors whose
RMS is at most 1 (the layer output, dx on the benchmark configurations) meet it literally.
Weight gradients with dy ~ N(0,1), and activation gradients of RMS well above 1, do not, and
cannot in bf16: they are sums of hundreds to thousands of products whose operands
(dg, du, dy*gate, act) are stored in bf16, their RMS is 1..17, and a 2^-9 relative error on
heavy-tailed operands leaves absolute errors of a few 1e-2 on elements that happen to be
small.  A CPU fp32 computation that rounds to bf16 at exactly the device's storage points
(the oracle's `emulate_bf16` mode, itself pinned on the CPU against an independent autograd
restatement with the same rounding points) shows the same violations.  So the rule is:

  1. norm-wise: ||got - ref||_F <= 1e-2 * ||ref||_F, always;
  2. the literal bound |got - ref| <= 1e-2 + 1e-2 * |ref| may be broken only as often as the
     bf16-emulating oracle breaks it: fraction(device) <= 1.5 * fraction(emulation) + 5/n (the
     device sits within 0-28 % of the emulation on every tensor measured; 5/n is small-count
     slack), never by more than a fixed share of the elements per class of tensor
     (STRICT_CEILING), and not at all when no emulation is given and rms(ref) <= 1;
     and wherever the emulation is given the device must sit close to it norm-wise
     (VS_EMULATION: 1.5e-3 for weight gradients), which is the sharp part of the rule;
  3. element-wise: |got - ref| <= 1e-2 * max(1, rms(ref)) + 1e-2 * |ref| for every element,
     unless the bf16-emulating oracle itself breaks that bound or comes within a hair of it, in
     which case the device may break it no more often than twice as often (plus one element:
     a frequency cannot be resolved below that) and by no more than 1.25x as far.

Every call appends its figures to the file named by the environment variable
MOE_PARITY_STATS (when set), one line per tensor, so that a GPU run leaves a record of how
far from the literal bound each tensor was.
"""
import os

RTOL = ATOL = 1e-2

# Largest fraction of elements allowed outside the LITERAL bound |d| <= 1e-2 + 1e-2*|ref|,
# whatever the emulation does.  The fraction grows with rms(ref): an element that happens to be
# small in a tensor of RMS 10 carries the absolute error of a tensor of RMS 10.  Largest values
# measured over all GPU tests (synthetic scales, dy ~ N(0,1)):
#   "act"    outputs and gradients of rows / activations / the residual stream: 0 wherever
#            rms(ref) <= 1; 9.8e-2 at rms(ref) = 12 (a 64 x 2048 case with weights ~ N(0, 0.08));
#   "wgrad"  expert and norm weight gradients (contractions over an expert's rows of bf16-stored
#            operands): 3.4e-2 on benchmark config 3 (rms 3), 1.2e-1 at rms(ref) = 16;
#   "token_sum" gradients that sum over ALL tokens: the router weight (differences of gate
#            gradients times x; rms 77 on config 3) and the pre-norm's weight: 2.1e-1 on config 3,
#            2.4e-1 at rms(ref) = 147 and 199.
STRICT_CEILING = {"act": 0.15, "wgrad": 0.20, "token_sum": 0.30}

# Largest norm-wise distance allowed between the device and the bf16-emulating oracle (brought to
# the device's output dtype).  The two round at the same points, so what separates them is fp32
# summation order, the hardware exp/rcp, and the rare one-ulp flip of a stored intermediate:
# measured 0.5e-4 to 3.7e-4 on expert weight gradients, up to 9e-4 on the router's, up to 4.9e-4
# on bf16 activation gradients (each entry against the emulation of its own rounding points:
# through `moe_ffn` the router path's gradient reaches x as a separate bf16 tensor).  This is the
# sharp check: 7 to 30 times tighter than the bar.
VS_EMULATION = {"act": 1.5e-3, "wgrad": 1.5e-3, "token_sum": 3e-3}


def klass_of(name: str) -> str:
    n = name.lower()
    if "dwr" in n or "router" in n or "dlogits" in n or "dgates" in n or "d norm" in n or "dbias" in n:
        return "token_sum"
    if "dw" in n or ".grad" in n or "weights" in n:
        return "wgrad"
    return "act"


def stats(got, ref, rtol=RTOL, atol=ATOL):
    got, ref = got.detach().float().cpu(), ref.detach().float().cpu()
    d = (got - ref).abs()
    rms = ref.pow(2).mean().sqrt().item()
    tol = atol * max(1.0, rms) + rtol * ref.abs()
    return {
        "n": d.numel(),
        "max_abs": d.max().item() if d.numel() else 0.0,
        "rms_ref": rms,
        "rel_fro": (d.norm() / ref.norm().clamp_min(1e-30)).item(),
        "frac_strict": (d > atol + rtol * ref.abs()).float().mean().item() if d.numel() else 0.0,
        "frac": (d > tol).float().mean().item() if d.numel() else 0.0,
        "worst": (d / tol).max().item() if d.numel() else 0.0,
    }


def _record(name, klass, s, e):
    path = os.environ.get("MOE_PARITY_STATS")
    if not path:
        return
    test = os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0]
    floor = "" if e is None else (f" floor_strict={e['frac_strict']:.3e} floor_scaled={e['frac']:.3e} "
                                  f"floor_worst={e['worst']:.2f} floor_rel_fro={e['rel_fro']:.3e} "
                                  f"device_vs_emulation_rel_fro={e['device_vs_emulation']:.3e}")
    with open(path, "a") as fh:
        fh.write(f"{test} | {name} [{klass}] n={s['n']} rms_ref={s['rms_ref']:.3e} rel_fro={s['rel_fro']:.3e} "
                 f"max_abs={s['max_abs']:.3e} outside_literal={s['frac_strict']:.3e} "
                 f"outside_rms_scaled={s['frac']:.3e} worst={s['worst']:.2f}{floor}\n")


def check(name, got, ref, ref_emulated=None, rtol=RTOL, atol=ATOL, say=print, klass=None):
    klass = klass or klass_of(name)
    s = stats(got, ref, rtol, atol)
    e = stats(ref_emulated, ref, rtol, atol) if ref_emulated is not None else None
    if e is not None:
        # how far the device is from the computation that rounds where it rounds (brought to the
        # device's output dtype): accumulation order, transcendental approximations and the odd
        # one-ulp flip of a stored intermediate are all that is left between the two
        em = ref_emulated.detach().cpu().to(got.dtype).float()
        e["device_vs_emulation"] = ((got.detach().float().cpu() - em).norm() / em.norm().clamp_min(1e-30)).item()
    _record(name, klass, s, e)
    line = (f"  {name}: max|d|={s['max_abs']:.3e} rms(ref)={s['rms_ref']:.3e} rel_fro={s['rel_fro']:.3e} "
            f"outside(strict)={s['frac_strict']:.2e} outside(rms-scaled)={s['frac']:.2e} worst={s['worst']:.2f}")
    assert s["rel_fro"] <= rtol, f"{name}: norm-wise error {s['rel_fro']:.3e} > {rtol}\n{line}"
    one = 1.0 / max(1, s["n"])  # a frequency cannot be resolved below one element
    if e is not None:
        allowed = min(STRICT_CEILING[klass], 1.5 * e["frac_strict"] + 5 * one)
    else:
        allowed = 0.0 if s["rms_ref"] <= 1.0 else STRICT_CEILING[klass]
    assert s["frac_strict"] <= allowed, (
        f"{name}: {s['frac_strict']:.3e} of the elements outside the literal bound, allowed {allowed:.3e} "
        f"(class {klass})\n{line}")
    if e is not None:
        assert e["device_vs_emulation"] <= VS_EMULATION[klass], (
            f"{name}: {e['device_vs_emulation']:.3e} away (norm-wise) from the bf16-emulating oracle, allowed "
            f"{VS_EMULATION[klass]:.1e} (class {klass})\n{line}")
    if s["frac"] == 0.0:
        say(line + "  OK")
        return s
    assert e is not None, f"{name}: outside tolerance and no bf16 floor given\n{line}"
    line += f" | bf16 floor: outside={e['frac']:.2e} worst={e['worst']:.2f}"
    assert s["frac"] <= 2 * e["frac"] + one + 1e-7 and s["worst"] <= 1.25 * max(1.0, e["worst"]), \
        f"{name}: worse than the bf16 storage floor\n{line}"
    say(line + "  OK (at the bf16 floor)")
    return s
