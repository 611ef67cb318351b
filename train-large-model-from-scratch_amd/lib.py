"""ctypes binding of libmoe_gfx950.so (the C ABI declared in include/moe_gfx950.h)."""
from __future__ import annotations

import ctypes
import os
import threading

from .build import LIB_PATH

_vp, _i64, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

# name -> (restype, argtypes); mirrors include/moe_gfx950.h one to one
SIGNATURES = {
    "moe_abi_version": (_int, []),
    "moe_router_topk_fwd": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_router_topk_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _int, _vp]),
    "moe_dispatch_workspace_bytes": (_i64, [_i64, _i64]),
    "moe_histogram_scan": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "moe_histogram_scan_checked": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "moe_static_scratch_bytes": (_i64, []),
    "moe_static_scratch_max_rows": (_i64, [_i64]),
    "moe_histogram_scan_static": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "moe_permute_fwd": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _vp]),
    "moe_permute_fwd_scatter": (_int, [_vp, _int, _vp, _i64, _i64, _i64, _vp, _vp]),
    "moe_permute_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _int, _vp]),
    "moe_permute_bwd_addend": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _vp, _int, _vp]),
    "moe_gemm_gateup_swiglu_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    "moe_gu_blocked_bytes": (_i64, [_i64, _i64, _i64]),
    "moe_gemm_gateup_swiglu_fwd_blocked": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_gemm_dgrad_down_swiglu_bwd_blocked": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _i64,
                                                      _vp, _vp]),
    "moe_gemm_force_row_tile": (_int, [_int]),
    "moe_gemm_down_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "moe_gemm_dgrad_down_swiglu_bwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_dgate_blocks": (_i64, [_i64]),
    "moe_gemm_dgrad_down_swiglu_bwd_dgate": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp,
                                                    _vp, _vp]),
    "moe_dgates_from_blocks": (_int, [_vp, _i64, _vp, _vp, _i64, _vp, _vp]),
    "moe_dgates_from_blocks_by_pos": (_int, [_vp, _i64, _vp, _vp, _i64, _vp, _vp]),
    "moe_gemm_dgrad_gateup": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "moe_gemm_wgrad": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _int, _int, _vp]),
    "moe_gemm_dgrad_down_swiglu_bwd_packed": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_gemm_dgrad_gateup_packed": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "moe_gemm_wgrad_pair": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _int, _int, _vp]),
    "moe_segment_offsets": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "moe_segments_by_length_max": (_i64, [_i64, _i64, _i64]),
    "moe_segment_offsets_by_length": (_int, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_wgrad_reduce_segments": (_int, [_vp, _vp, _i64, _i64, _i64, _vp, _int, _int, _vp]),
    "moe_combine_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _int, _vp]),
    "moe_combine_bwd": (_int, [_vp, _int, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_combine_fwd_residual": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _int, _vp]),
    "moe_rmsnorm_fwd": (_int, [_vp, _int, _vp, ctypes.c_float, _i64, _i64, _vp, _vp, _vp]),
    "moe_rmsnorm_router_supported": (_int, [_i64, _i64, _i64]),
    "moe_rmsnorm_router_fwd": (_int, [_vp, _int, _vp, ctypes.c_float, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp,
                                      _vp, _vp, _vp]),
    "moe_rmsnorm_bwd_workspace_bytes": (_i64, [_i64, _i64]),
    "moe_rmsnorm_bwd": (_int, [_vp, _int, _vp, _vp, _vp, _int, _vp, _vp, _i64, _i64, _vp, _vp, _vp,
                               _i64, _vp]),
    "moe_combine_bwd_by_token": (_int, [_vp, _int, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_cast_f32_bf16": (_int, [_vp, _vp, _i64, _vp]),
    "moe_ffn_forward_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64, _i64]),
    "moe_ffn_forward": (_int, [_vp, _int, _vp, _int, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _int,
                                _vp, _i64, _vp]),
    "moe_f32_gather_rows": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "moe_f32_combine_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "moe_f32_combine_bwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _vp, _vp]),
    "moe_f32_permute_bwd": (_int, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "moe_f32_swiglu_fwd": (_int, [_vp, _vp, _i64, _vp, _vp]),
    "moe_f32_swiglu_bwd": (_int, [_vp, _vp, _vp, _i64, _vp, _vp, _vp]),
    "moe_f32_gemm_rows": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp, _int, _vp]),
    "moe_f32_gemm_wgrad": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _int, _vp]),
    "moe_f32_gemm_force_tile": (_int, [_int]),
}

ERRORS = {-1: "MOE_ERR_NULL", -2: "MOE_ERR_SHAPE", -3: "MOE_ERR_LIMIT", -4: "MOE_ERR_DTYPE",
          -5: "MOE_ERR_WORKSPACE", -6: "MOE_ERR_ALIGN"}

DT_BF16, DT_F32 = 0, 1


class MoELibError(RuntimeError):
    pass


class MoELib:
    def __init__(self, path: str):
        self.path = path
        self.cdll = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(self.cdll, name)  # AttributeError if the symbol is missing
            fn.restype, fn.argtypes = res, args
        self.abi_version = self.cdll.moe_abi_version()
        # Optional observer of the launches (a profiling aid): an object with before(name) and
        # after(name), called around every entry point, e.g. to record events on the stream.
        self.observer = None

    def call(self, name: str, *args):
        obs = self.observer
        if obs is not None:
            obs.before(name)
        rc = getattr(self.cdll, name)(*args)
        if obs is not None:
            obs.after(name)
        if rc != 0:
            what = ERRORS.get(rc, f"hipError_t {rc}" if rc > 0 else f"code {rc}")
            raise MoELibError(f"{name} failed: {what}")


_lock = threading.Lock()
_lib: MoELib | None = None


def load() -> MoELib:
    """Load the built library.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:  # the usual case, without the lock
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise MoELibError(
                    f"{LIB_PATH} is not built; run `python __graft_entry__.py` "
                    "(or train-large-model-from-scratch_amd/build.py) first")
            import torch  # noqa: F401  -- makes sure torch's HIP runtime is the one in the process
            _lib = MoELib(LIB_PATH)
        return _lib
