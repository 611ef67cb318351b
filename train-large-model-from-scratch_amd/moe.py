"""`MoE`: drop-in for the reference's module of the same name (model/modules/mlp.py:47-169).

Same constructor, attribute names, parameter names / shapes / dtype / init seeding, and the
same `forward(x) -> (out, gate_logits)` contract, so `Block` (model/gpt.py:19-34) and the
trainer can use it unchanged.  Inside, everything after the router linear runs in the
gfx950 kernels of libmoe_gfx950.so.
"""
from __future__ import annotations

import torch
import torch.nn as nn
from torch.optim.optimizer import register_optimizer_step_post_hook

from . import ops, parallel_state, traced
from .functional import moe_ffn, moe_ffn_f32, prenorm_moe, routed_moe, router_linear


# Number of optimizer steps taken in this process, counted by a global post-step hook of
# torch.optim: one of the signs that master weights may have changed (see MoE._bf16_operands).
# The hook is installed when the first MoE that caches its weight copies is built, not at import.
_optimizer_steps = [0]
_hook_handle = []


def _count_optimizer_step(optimizer, args, kwargs):
    _optimizer_steps[0] += 1


def _install_step_counter():
    if not _hook_handle:
        _hook_handle.append(register_optimizer_step_post_hook(_count_optimizer_step))


class MoE(nn.Module):
    def __init__(self, config, top_k: int | None = None):
        super().__init__()
        # mlp.py:50 uses torch.cuda.current_device(); a CPU fallback exists only so that the
        # constructor contract (names, shapes, seeding) can be checked without a GPU.
        # forward() has no CPU path.
        self.device = torch.cuda.current_device() if torch.cuda.is_available() else torch.device("cpu")
        self.config = config
        self.num_experts = config.num_experts
        self.top_k = top_k if top_k is not None else config.num_experts_per_tok
        assert self.top_k <= self.num_experts, (
            f"top_k must be less than or equal to num_experts, got {self.top_k} and {self.num_experts}")
        self.hidden_size = config.hidden_size
        self.intermediate_size = config.moe_intermediate_size
        # The reference's flag says whether torch's F.grouped_mm branch is taken
        # (mlp.py:57-63); it is False on ROCm.  The grouped GEMM here is the library's own.
        self.grouped_gemm_supported = False

        self.router = nn.Linear(self.hidden_size, self.num_experts, bias=False, device=self.device)

        self.ep_size = parallel_state.get_ep_world_size()
        assert self.num_experts % self.ep_size == 0
        self.num_local_experts = self.num_experts // self.ep_size

        E, I, H = self.num_local_experts, self.intermediate_size, self.hidden_size
        self.experts_gate_weights = nn.Parameter(torch.empty(E, I, H, device=self.device))
        self.experts_up_weights = nn.Parameter(torch.empty(E, I, H, device=self.device))
        self.experts_down_weights = nn.Parameter(torch.empty(E, H, I, device=self.device))
        self.experts_act_fn = nn.SiLU()
        self._shadow = {}  # name -> (key of the master's state, bf16 copy); not part of state_dict
        # False: cast the fp32 masters in every forward, as the reference does (no cached copies,
        # nothing that a write through `.data` could leave stale).
        self.cache_bf16_weights = True
        # True: before every use of a cached copy, 64 of its elements are compared with the
        # master (one small gather and a host synchronisation per stack) and a stale copy raises.
        self.verify_weight_cache = False
        _install_step_counter()
        # Opt-in: expert weight gradients are added to `.grad` by the kernel that computes them
        # instead of by autograd (saves a pass over them per gradient-accumulation micro-step;
        # hooks on these three parameters then do not run, see functional.py).
        self.accumulate_wgrad_into_grad = False
        # False: `forward_prenorm` takes the router logits from the library's product (the one
        # `forward` uses) instead of the fused norm+router kernel, whose summation order can move
        # a bf16 logit by one unit in the last place and with it the routing of a near-tie.
        self.fused_router = True
        # False (the reference's rule): a call without autocast on fp32 input and fp32 parameters
        # computes in fp32 from end to end, as the reference's bmm's then do (mlp.py:154-157).
        # True: such a call runs on the bf16 matrix cores like every other one (fp32 in and out,
        # bf16 operands, fp32 accumulation): eight times the throughput, at bf16 precision.
        self.bf16_compute_for_fp32_calls = False
        self._init_expert_weights(config.seed)

    def _init_expert_weights(self, base_seed: int):
        """Seeding contract of mlp.py:77-93: expert e draws gate, up, down (in that order) from
        a generator seeded with base_seed + global expert index; the router from base_seed."""
        first = parallel_state.get_ep_rank() * self.num_local_experts
        std = self.config.init_std
        stacks = (self.experts_gate_weights, self.experts_up_weights, self.experts_down_weights)
        dev = self.experts_gate_weights.device
        fork_devices = [dev] if dev.type == "cuda" else []
        with torch.random.fork_rng(devices=fork_devices):
            for local in range(self.num_local_experts):
                torch.manual_seed(base_seed + first + local)
                for stack in stacks:
                    nn.init.normal_(stack[local], mean=0.0, std=std)
        with torch.random.fork_rng(devices=fork_devices):
            torch.manual_seed(base_seed)
            nn.init.normal_(self.router.weight, mean=0.0, std=std)

    def invalidate_weight_cache(self):
        """Drop the bf16 copies of the expert weights; the next forward casts them again.
        Needed only after the masters were rewritten through `.data` outside an optimizer
        step (see `_bf16_operands`)."""
        self._shadow.clear()

    def _bf16_operands(self):
        """bf16 copies of the fp32 master weights for the matrix cores.  The reference pays
        three fp32->bf16 casts per forward (autocast cannot cache the transposed views of
        mlp.py:154-157); here gradient-accumulation micro-steps share one cast.  A copy is
        redone when its master may have changed, i.e. when any of these moved since the cast:
          - the master's tensor version (every in-place update under `no_grad`, `copy_` of
            `load_state_dict`, ...),
          - the count of `torch.optim` optimizer steps in this process (a global post-step
            hook): the reference's ZeRO-1 wrapper steps an inner torch optimizer and then
            broadcasts through `p.data` (distributed_optimizer.py:85-94, :119), which the
            version counter does not see,
          - the master's storage or device.
        Writes through `.data` with no `torch.optim` step in between (an EMA swap, a manual
        `p.data.copy_`, an optimizer that is not a `torch.optim.Optimizer`) are the one case this
        cannot see: `invalidate_weight_cache()` is there for them, `cache_bf16_weights = False`
        turns the cache off, and `verify_weight_cache = True` detects a stale copy.  The copies are handed to the
        expert function together with the masters: the masters receive the gradients.
        While the stream is being captured into a graph the cache is neither read nor written: the
        casts are recorded with the rest of the step, so every replay rounds the masters as they
        are then (a copy that was fresh at capture time would be stale after the first optimizer
        step, and no Python runs at a replay to notice)."""
        out = []
        capturing = torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()
        for name in ("experts_gate_weights", "experts_up_weights", "experts_down_weights"):
            w = getattr(self, name)
            if w.dtype == torch.bfloat16:
                out.append(None)
                continue
            if not self.cache_bf16_weights or capturing:
                out.append(None)  # the expert function casts
                continue
            key = (w._version, _optimizer_steps[0], w.data_ptr(), w.device)
            held = self._shadow.get(name)
            if held is None or held[0] != key:
                held = (key, ops.cast_bf16(w.detach().contiguous()))
                self._shadow[name] = held
            elif self.verify_weight_cache:
                idx = torch.randint(0, w.numel(), (64,), device=w.device)
                if not torch.equal(w.detach().reshape(-1)[idx].to(torch.bfloat16), held[1].reshape(-1)[idx]):
                    raise RuntimeError(
                        f"MoE: the cached bf16 copy of {name} no longer matches its fp32 master (the master "
                        "was rewritten without an optimizer step or a version bump); call "
                        "invalidate_weight_cache() after such writes or set cache_bf16_weights = False")
            out.append(held[1])
        return out

    @torch._dynamo.disable  # opaque to torch.compile, like the reference's own a2a op (comm.py:42)
    def _experts(self, x2d: torch.Tensor, logits2d: torch.Tensor) -> torch.Tensor:
        return moe_ffn(x2d, logits2d, self.experts_gate_weights, self.experts_up_weights,
                       self.experts_down_weights, self.top_k, bf16_weights=self._bf16_operands(),
                       accumulate_into_grad=self.accumulate_wgrad_into_grad)

    @torch._dynamo.disable
    def _layer(self, x2d: torch.Tensor):
        return routed_moe(x2d, self.router.weight, self.experts_gate_weights, self.experts_up_weights,
                          self.experts_down_weights, self.top_k, bf16_weights=self._bf16_operands(),
                          accumulate_into_grad=self.accumulate_wgrad_into_grad)

    def _router_has_hooks(self) -> bool:
        r = self.router
        return bool(r._forward_hooks or r._forward_pre_hooks or r._backward_hooks or r._backward_pre_hooks)

    def _router_in_bf16(self, x: torch.Tensor) -> bool:
        """Whether `self.router(x)` would be a bf16 product anyway (bf16 autocast, or bf16
        tensors): then router and experts run as one autograd node."""
        if x.dtype == torch.bfloat16 and self.router.weight.dtype == torch.bfloat16:
            return True
        return (x.is_cuda and torch.is_autocast_enabled("cuda")
                and torch.get_autocast_dtype("cuda") == torch.bfloat16)

    def _runs_in_fp32(self, x: torch.Tensor) -> bool:
        """Whether the reference would run this call in fp32: fp32 input, fp32 parameters, no
        autocast."""
        if self.bf16_compute_for_fp32_calls or x.dtype != torch.float32:
            return False
        if x.is_cuda and torch.is_autocast_enabled("cuda"):
            return False
        return all(w.dtype == torch.float32 for w in (self.router.weight, self.experts_gate_weights,
                                                      self.experts_up_weights, self.experts_down_weights))

    @staticmethod
    @torch._dynamo.disable
    def _experts_f32(x2d, logits2d, w1, w3, w2, k) -> torch.Tensor:
        return moe_ffn_f32(x2d, logits2d, w1, w3, w2, k)

    def forward(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        B, T, D = x.size()
        if self._runs_in_fp32(x):
            gate_logits = self.router(x)  # fp32 product and fp32 gradients, as nn.Linear gives them
            ffn = traced.moe_ffn_f32 if torch.compiler.is_compiling() else self._experts_f32
            out = ffn(x.reshape(B * T, D), gate_logits.reshape(B * T, self.num_experts),
                      self.experts_gate_weights, self.experts_up_weights, self.experts_down_weights, self.top_k)
            return out.reshape(B, T, D), gate_logits
        if torch.compiler.is_compiling():
            # under torch.compile (trainer.py:130-131): the same kernels as registered
            # operators the tracer can keep in the graph (traced.py); no cached weight copies
            if self._router_in_bf16(x):
                out, gate_logits = traced.routed_moe(x.reshape(B * T, D), self.router.weight,
                                                     self.experts_gate_weights, self.experts_up_weights,
                                                     self.experts_down_weights, self.top_k)
                return out.reshape(B, T, D), gate_logits.reshape(B, T, self.num_experts)
            gate_logits = nn.functional.linear(x, self.router.weight)
            out = traced.moe_ffn(x.reshape(B * T, D), gate_logits.reshape(B * T, self.num_experts),
                                 self.experts_gate_weights, self.experts_up_weights,
                                 self.experts_down_weights, self.top_k)
            return out.reshape(B, T, D), gate_logits
        if self._router_has_hooks():
            # hooks on the nn.Linear fire only if it is called: the product is the module's own
            # (mlp.py:100), the logits go to the expert function as in the reference
            gate_logits = self.router(x)
            out = self._experts(x.reshape(B * T, D), gate_logits.reshape(B * T, self.num_experts))
            return out.reshape(B, T, D), gate_logits
        if self._router_in_bf16(x):
            out, gate_logits = self._layer(x.reshape(B * T, D))
            return out.reshape(B, T, D), gate_logits.reshape(B, T, self.num_experts)
        # [B, T, E] in the dtype nn.Linear would give (mlp.py:100).  `self.router` holds the
        # parameter; the product goes through router_linear for its faster weight gradient
        gate_logits = router_linear(x, self.router.weight)
        out = self._experts(x.reshape(B * T, D), gate_logits.reshape(B * T, self.num_experts))
        return out.reshape(B, T, D), gate_logits

    @torch._dynamo.disable
    def forward_prenorm(self, x: torch.Tensor, norm: nn.Module, add_residual: bool = True):
        """`x + self(norm(x))[0]` and the router logits in one call, for a caller that owns the
        pre-norm and the residual add (model/gpt.py:32-33).  `norm` is the caller's RMSNorm
        module (`weight`, `variance_epsilon`; model/modules/norm.py:6-19).  Results match
        calling the three pieces separately under bf16 autocast; the residual stream is read
        once on the way in and written once on the way out."""
        B, T, D = x.size()
        if D > 8192 or self._router_has_hooks() or self._runs_in_fp32(x):
            # wider than the fused norm kernels hold in registers, hooks on the router that only a
            # call of the nn.Linear runs, or an fp32 call (the norm then is the caller's fp32
            # module): the separate calls
            out, logits = self(norm(x))
            return (x + out if add_residual else out), logits
        out, logits = prenorm_moe(x.reshape(B * T, D), norm.weight, self.router.weight,
                                  self.experts_gate_weights, self.experts_up_weights,
                                  self.experts_down_weights, self.top_k, eps=norm.variance_epsilon,
                                  add_residual=add_residual, bf16_weights=self._bf16_operands(),
                                  accumulate_into_grad=self.accumulate_wgrad_into_grad,
                                  fused_router=self.fused_router)
        return out.reshape(B, T, D), logits.reshape(B, T, self.num_experts)
