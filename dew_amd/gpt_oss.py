"""GPT-OSS's biased router and interleaved experts with the clamped 1.702 gating, on the gfx950 HIP kernels:
the host-side mirror of the reference's `dew.nn.gpt_oss` (src/dew/nn/gpt_oss.py:49-171), forward only, with the
same names, fields and parameter tree:

    params/router/{kernel [D, E], bias [E]}                     fp32
    params/experts/{gate_up_proj_bias [E, 2F], down_proj_bias [E, D]}
    quantization/experts/{gate_up_proj, down_proj}              quantized banks [E, D, 2F] and [E, F, D]

The fused `gate_up_proj` holds gate in its even columns and up in its odd ones; one launch multiplies it, adds
the bias, clamps and gates (`ops.gateup_interleaved`). The final `sum(slots * weights)` keeps the router's
weights in fp32 and rounds once, which is at least as accurate as a bf16 sum of bf16 products.
"""

import dataclasses

import torch

from . import gemm, ops
from .moe import Gathered, _Module, _at, _implementation, _sorted_locally, expert_matrix, expert_projection, rounded_operand

SWIGLU_LIMIT = 7.0
"""The clamp of `swiglu_clamped(..., 7.0)` (src/dew/nn/gpt_oss.py:120)."""


@dataclasses.dataclass(frozen=True)
class GptOssExperts(_Module):
    """Interleaved gate/up matrices with the clamped 1.702 gating (src/dew/nn/gpt_oss.py:49-126)."""

    hidden_size: int
    intermediate_size: int
    num_local_experts: int
    implementation: str = "auto"
    dispatch: str = "auto"
    capacity_factor: float | None = None
    dtype: torch.dtype | None = None
    precision: object = None

    def __post_init__(self):
        if self.dispatch not in ("auto", "global"):
            raise ValueError(f"dispatch {self.dispatch!r}: one device sorts its slots locally ('global')")
        if self.capacity_factor is not None:
            raise ValueError("capacity dropping is not part of the HIP experts")

    def model_flops(self, rows: int) -> float:
        """Three maps per expert assignment (src/dew/nn/gpt_oss.py:63-68)."""
        return 3 * 2.0 * rows * self.hidden_size * self.intermediate_size

    def _leaf(self, name: str):
        found = _at(self.variables.get("params"), (*self.path, name))
        if found is None:
            raise KeyError(f"no params/{'/'.join(self.path)}/{name}")
        return found

    def _project(self, tokens: Gathered, sizes, parameters) -> torch.Tensor:
        """src/dew/nn/gpt_oss.py:106-126: each bias meets its expert's rows' sums before their one rounding."""
        gate_up, gate_bias, down, down_bias = parameters
        compute = torch.bfloat16 if self.dtype is None else self.dtype
        activated = gemm.gemm(tokens.tokens, gate_up, sizes, gather=tokens.rows, epilogue="gpt_oss_gated",
                              epilogue_operands=(rounded_operand(gate_bias, compute), SWIGLU_LIMIT), compute=compute,
                              out_dtype=compute, implementation=_implementation(self.implementation))
        return expert_projection(activated, down, sizes, self.dtype, self.implementation, self.precision, bias=down_bias,
                                 scatter=tokens.slots)

    def __call__(self, x: torch.Tensor, weights: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        if weights.shape != indices.shape:
            raise ValueError(f"routing {tuple(indices.shape)} does not describe weights {tuple(weights.shape)}")
        parameters = (expert_matrix(self.variables, self.path, "gate_up_proj"), self._leaf("gate_up_proj_bias"),
                      expert_matrix(self.variables, self.path, "down_proj"), self._leaf("down_proj_bias"))
        tokens = x.reshape(-1, x.shape[-1]).contiguous()
        top_k = indices.shape[-1]
        plan, sizes = _sorted_locally(indices, self.num_local_experts)
        slots = self._project(Gathered(tokens, plan.rows, plan.order), sizes, parameters)
        out = ops.combine(slots.reshape(tokens.shape[0], top_k, self.hidden_size), weights.reshape(-1, top_k).contiguous())
        return out.reshape(*x.shape[:-1], self.hidden_size)


@dataclasses.dataclass(frozen=True)
class GptOssMLP(_Module):
    """Softmax over the selected biased logits, then the selected expert sum (src/dew/nn/gpt_oss.py:129-171)."""

    hidden_size: int
    intermediate_size: int
    num_local_experts: int
    num_experts_per_tok: int
    implementation: str = "auto"
    dispatch: str = "auto"
    capacity_factor: float | None = None
    dtype: torch.dtype | None = None
    precision: object = None

    @property
    def routes_experts(self) -> bool:
        return True

    @property
    def experts(self) -> GptOssExperts:
        return GptOssExperts(self.hidden_size, self.intermediate_size, self.num_local_experts, self.implementation,
                             self.dispatch, self.capacity_factor, self.dtype,
                             self.precision)._bound(self.variables, (*self.path, "experts"))

    def logits(self, x: torch.Tensor) -> torch.Tensor:
        """The biased router's fp32 logits (src/dew/nn/gpt_oss.py:160-165)."""
        router = _at(self.variables["params"], (*self.path, "router"))
        flat = x.reshape(-1, x.shape[-1]).contiguous()
        return ops.router_logits(flat, router["kernel"], router["bias"]).reshape(*x.shape[:-1], self.num_local_experts)

    def __call__(self, x: torch.Tensor, routes=None) -> torch.Tensor:
        if routes is not None:
            raise ValueError("replayed routing is not part of the HIP router")
        # top_k of the logits, then the softmax of the chosen logits alone (`renormalized_softmax`,
        # src/dew/nn/moe.py:194-199): the softmax router's choice and renormalized weights
        weights, indices = ops.route(self.logits(x).reshape(-1, self.num_local_experts), self.num_experts_per_tok,
                                     score_function="softmax", normalize_weights=True)
        return self.experts(x, weights.reshape(*x.shape[:-1], -1), indices.reshape(*x.shape[:-1], -1))
