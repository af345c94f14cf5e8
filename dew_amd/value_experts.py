"""Routed value experts: an attention layer's values as a mixture of projections (K2 Horizon's MoVA), the host-side
mirror of the reference's `ValueExperts` / `RoutedValues` (src/dew/nn/value_experts.py:34-98). `top_k` of `experts`
projections of the hidden state per token, each through a SiLU, summed under the router's weights in fp32: the routed
MLP's own launches (router, dispatch sort, one grouped product scattered to slot order, combine) with the stand-alone
activation between the product and the combine.

Parameters, as the reference names them: `<path>/v_router/kernel [in_features, experts]` fp32 (with `bias`, the
selection bias at `moe/<path>/v_router/e_score_correction_bias`) and `<path>/v_proj/kernel [experts, in_features,
features]`, a bf16 tensor or a bank of `dew_amd.formats`."""

import dataclasses

import torch

from . import ops
from .gemm import GroupSizes
from .moe import Gathered, Router, _Module, expert_matrix, expert_projection


@dataclasses.dataclass(frozen=True)
class ValueExperts:
    """A layer's routed value experts (src/dew/nn/value_experts.py:34-51)."""

    experts: int
    top_k: int
    score_function: str = "sigmoid"
    norm_topk_prob: bool = True
    scaling: float = 1.0
    bias: bool = False

    def __post_init__(self):
        if not 0 < self.top_k <= self.experts:
            raise ValueError(f"value experts choose top_k of their experts, got {self.top_k} of {self.experts}")


@dataclasses.dataclass(frozen=True)
class RoutedValues(_Module):
    """`spec`'s value experts over hidden states `[..., in_features]` (src/dew/nn/value_experts.py:58-98)."""

    spec: ValueExperts
    in_features: int
    features: int
    implementation: str = "auto"

    @property
    def router(self) -> Router:
        spec = self.spec
        return Router(spec.experts, self.in_features, spec.top_k, spec.score_function, spec.norm_topk_prob, spec.scaling,
                      expert_bias=spec.bias)._bound(self.variables, (*self.path, "v_router"))

    def __call__(self, x: torch.Tensor, *, logits: torch.Tensor | None = None) -> torch.Tensor:
        """`logits`, where given, are the router's (a test's own); else the router's kernel multiplies the tokens."""
        router = self.router
        weights, indices = router(x) if logits is None else router.routed(logits)
        tokens = x.reshape(-1, x.shape[-1]).contiguous()
        top_k = indices.shape[-1]
        plan = ops.sort_by_expert(indices.reshape(-1, top_k), self.spec.experts)
        kernel = expert_matrix(self.variables, (*self.path, "v_proj"))
        projected = expert_projection(Gathered(tokens, plan.rows, plan.order), kernel, GroupSizes(plan.sizes, plan.offsets), None,
                                      self.implementation, scatter=plan.order)
        slots = ops.silu(projected).reshape(tokens.shape[0], top_k, self.features)
        out = ops.combine(slots, weights.reshape(-1, top_k).contiguous())
        return out.reshape(*x.shape[:-1], self.features)
