"""Peak-throughput table and MFU helpers for AMD Instinct parts, in the shape of the reference's
`utils/profile.py` (`GPU_PEAK_FLOPS` :3-19, `get_gpu_peak_flops` :22-36, `compute_mfu` :38-48),
whose table knows NVIDIA parts only: on an MI355X its trainer's MFU line prints 0 with a warning.
`GPU_PEAK_FLOPS` here can be merged into the reference's dict (`GPU_PEAK_FLOPS.update(...)`); the
two functions keep the reference's names, arguments and return values.

Figures are the vendor's dense (no structured sparsity) matrix peaks in FLOP/s.
"""
from __future__ import annotations

import torch

GPU_PEAK_FLOPS = {
    "MI355X": {"fp32": 157.3e12, "fp16": 2.5e15, "bf16": 2.5e15, "fp8": 5.0e15},
    "MI350X": {"fp32": 144.2e12, "fp16": 2.3e15, "bf16": 2.3e15, "fp8": 4.6e15},
    "MI325X": {"fp32": 163.4e12, "fp16": 1307.4e12, "bf16": 1307.4e12, "fp8": 2614.9e12},
    "MI300X": {"fp32": 163.4e12, "fp16": 1307.4e12, "bf16": 1307.4e12, "fp8": 2614.9e12},
}


def peak_for_device_name(gpu_name: str, dtype: str = "bf16") -> float:
    """Peak FLOP/s for a device name as `torch.cuda.get_device_name` reports it (0 if unknown)."""
    dtype = dtype.lower()
    for key, row in GPU_PEAK_FLOPS.items():
        if key in gpu_name:
            return float(row.get(dtype, 0) or 0)
    return 0.0


def get_gpu_peak_flops(dtype: str = "bf16", per_device: bool = True) -> float:
    """utils/profile.py:22-36 for AMD parts: peak FLOP/s of device 0's type (times the device
    count unless `per_device`)."""
    gpu_name = torch.cuda.get_device_name(0)
    peak = peak_for_device_name(gpu_name, dtype)
    if peak == 0:
        print(f"Warning: unknown or unsupported FLOPs for GPU {gpu_name} with dtype {dtype}")
    return peak if per_device else peak * torch.cuda.device_count()


def compute_mfu(model, batch_size, seq_len, time, ga: int = 1, dtype: str = "bf16"):
    """utils/profile.py:38-48: (mfu, achieved FLOP/s, peak FLOP/s) from the model's own
    `get_flops_per_fwd_bwd` (model/gpt.py:78-98)."""
    total_flops = model.get_flops_per_fwd_bwd(batch_size, seq_len) * ga
    actual = total_flops / time if time > 0 else 0.0
    peak = get_gpu_peak_flops(dtype=dtype, per_device=True)
    return (actual / peak if peak else 0), actual, peak
