"""Writes tests/golden/oracle_tiny.npz: seeded tiny inputs and what oracle/moe_oracle.py computes
from them (fp32 mode and bf16-rounding mode, forward and backward).  The file is a tripwire for
the oracle itself: tests/test_oracle.py recomputes and compares, so an edit that changes what the
oracle computes (in particular where its bf16-rounding mode rounds) has to come with a
regenerated fixture and shows up in review.  It is produced by this repository's own oracle, not
by the reference (which ships no fixtures for this path and was not run).

    python tests/golden/make_oracle_fixture.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import moe_oracle as O  # noqa: E402

T, H, E, I, K = 24, 32, 4, 24, 2
KEYS_F = ("out", "g", "u", "act", "y", "gates")
KEYS_B = ("dx", "dw1", "dw3", "dw2", "dwr", "dgates", "dlogits", "dxp", "dg", "du")


def inputs():
    g = torch.Generator().manual_seed(20240607)
    rb = lambda t: t.to(torch.bfloat16).float()
    x = rb(torch.randn(T, H, generator=g))
    wr = rb(torch.randn(E, H, generator=g) * 0.3)
    w1 = rb(torch.randn(E, I, H, generator=g) * 0.2)
    w3 = rb(torch.randn(E, I, H, generator=g) * 0.2)
    w2 = rb(torch.randn(E, H, I, generator=g) * 0.2)
    dy = rb(torch.randn(T, H, generator=g))
    logits = rb(torch.nn.functional.linear(x, wr))
    return x, wr, w1, w3, w2, dy, logits


def compute():
    x, wr, w1, w3, w2, dy, logits = inputs()
    rec = {"x": x, "wr": wr, "w1": w1, "w3": w3, "w2": w2, "dy": dy, "logits": logits}
    for tag, emu in (("f32", False), ("emu", True)):
        f = O.moe_forward(x, wr, w1, w3, w2, K, logits=logits, emulate_bf16=emu)
        b = O.moe_backward(f, dy, wr, w1, w3, w2, emulate_bf16=emu)
        if not emu:
            rec["ids"] = torch.from_numpy(f["ids"])
            rec["pos_to_row"] = torch.from_numpy(f["pos_to_row"])
            rec["counts"] = torch.from_numpy(f["counts"])
        for k in KEYS_F:
            rec[f"{tag}_{k}"] = f[k]
        for k in KEYS_B:
            rec[f"{tag}_{k}"] = b[k]
    return {k: v.numpy() for k, v in rec.items()}


if __name__ == "__main__":
    np.savez_compressed(os.path.join(HERE, "oracle_tiny.npz"), **compute())
    print("wrote", os.path.join(HERE, "oracle_tiny.npz"))
