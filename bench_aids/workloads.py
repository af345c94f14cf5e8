"""The five benchmark workloads: their shapes, router settings and seeded synthetic inputs, at full or reduced size.

Read by bench.py (what it measures), by the parity tests (the same cases, mostly reduced) and by the smoke run.
"""

import dataclasses

import numpy as np
import torch

from dew_amd import codecs, formats


@dataclasses.dataclass(frozen=True)
class Case:
    name: str
    tokens: int
    d_model: int
    d_ff: int
    experts: int
    top_k: int
    quant: str                      # fp8_channel | fp8_block | mxfp4 | nvfp4
    router: dict
    logit_bias_std: float = 0.0     # per-expert bias added to the logits (load imbalance)
    shared: bool = False

    def scaled(self, **changes) -> "Case":
        return dataclasses.replace(self, **changes)


SOFTMAX = dict(score_function="softmax", normalize_weights=True)
DEEPSEEK = dict(score_function="sigmoid", normalize_weights=True, routed_scaling_factor=2.5, expert_groups=8,
                groups_per_token=4)

CONFIGS = {
    "c1": Case("c1", 2048, 512, 1024, 8, 2, "fp8_channel", SOFTMAX),
    "c2": Case("c2", 16384, 4096, 14336, 8, 2, "mxfp4", SOFTMAX, logit_bias_std=0.5),
    "c3": Case("c3", 64, 2048, 768, 128, 8, "fp8_block", SOFTMAX),
    "c4": Case("c4", 8192, 7168, 2048, 256, 8, "fp8_block", DEEPSEEK, shared=True),
    "c5": Case("c5", 4096, 4096, 14336, 8, 2, "nvfp4", SOFTMAX),
}


def quantize(weight: torch.Tensor, quant: str):
    """`weight [E, K, N]` fp32 as the bank `quant` names, in the reference's storage layout."""
    if quant == "fp8_channel":
        return formats.Fp8Channels.quantized(weight)
    if quant == "fp8_block":
        return formats.Fp8Blocks.quantized(weight)
    if quant == "nvfp4":
        return formats.NvFp4.quantized(weight)
    if quant == "mxfp4":
        blocks, scales = codecs.quantize_mxfp4(weight)
        powers = codecs.mxfp4_tensor_powers(blocks, scales)
        assert powers is not None, "an N(0, 0.02) bank's group powers fit E4M3"
        return formats.NvFp4.of(*codecs.mxfp4_as_nvfp4(blocks, scales, powers))
    if quant == "bf16":
        return formats.Bf16(weight.to(torch.bfloat16))
    raise ValueError(quant)


def inputs(case: Case, seed: int = 0):
    """Host tensors of one case: activations (bf16), router logits, selection bias, banks (reference layout)."""
    rng = np.random.default_rng(seed)
    x = torch.from_numpy(rng.standard_normal((case.tokens, case.d_model)).astype(np.float32)).to(torch.bfloat16)
    logits = rng.standard_normal((case.tokens, case.experts)).astype(np.float32)
    if case.logit_bias_std:
        logits = logits + (rng.standard_normal(case.experts) * case.logit_bias_std).astype(np.float32)
    bias = None
    if case.router.get("score_function") == "sigmoid":
        bias = torch.from_numpy((rng.standard_normal(case.experts) * 0.05).astype(np.float32))

    def bank(depth, width, experts=case.experts):
        weight = torch.from_numpy((rng.standard_normal((experts, depth, width)) * 0.02).astype(np.float32))
        return quantize(weight, case.quant)

    banks = dict(gate=bank(case.d_model, case.d_ff), up=bank(case.d_model, case.d_ff), down=bank(case.d_ff, case.d_model))
    shared = None
    if case.shared:
        shared = dict(gate=bank(case.d_model, case.d_ff, 1), up=bank(case.d_model, case.d_ff, 1),
                      down=bank(case.d_ff, case.d_model, 1))
    return dict(x=x, logits=torch.from_numpy(logits), bias=bias, banks=banks, shared=shared)
