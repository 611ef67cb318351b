"""MI355X-native MoE expert path (drop-in for the reference's model/modules/mlp.py::MoE)."""
from . import configs, lib, ops, parallel_state, profile  # noqa: F401
from .config import ModelConfig  # noqa: F401
from .functional import experts_rows, experts_rows_f32, moe_ffn, moe_ffn_f32, prenorm_moe, routed_moe, router_linear  # noqa: F401
from .moe import MoE  # noqa: F401
from .block import Block  # noqa: F401
