"""Test infrastructure, not product code: the oracle's decoding of a bank held as one of dew_amd.formats' types.

Only the tests, the smoke run and bench.py's CPU-baseline leg call this (the product never imports the oracle).
"""

import numpy as np

from dew_amd import formats


def dequantized(bank):
    """(values `[E, K, N]` fp32 as the reference's load decodes them, per-expert accumulator factor or None),
    by the oracle's decoders."""
    from oracle import moe_oracle as oracle

    if isinstance(bank, formats.NvFp4):
        words = bank.words.cpu().numpy().view(np.uint32)
        return oracle.nvfp4_bank_decoded(words, bank.scales.cpu().numpy()), oracle.nvfp4_bank_factor(bank.scale.cpu().numpy())
    if isinstance(bank, formats.Fp8Blocks):
        return oracle.dequantize_fp8_blocks(bank.codes.cpu().numpy(), bank.scale_inv.cpu().numpy()), None
    if isinstance(bank, formats.Fp8Channels):
        return oracle.dequantize_fp8_channels(bank.codes.cpu().numpy(), bank.scales.cpu().numpy()), None
    if isinstance(bank, formats.Bf16):
        return bank.weights.float().cpu().numpy(), None
    if isinstance(bank, formats.Mxfp4Blocks):
        return oracle.decode_mxfp4(bank.blocks.cpu().numpy(), bank.scales.cpu().numpy()), None
    raise TypeError(type(bank))
