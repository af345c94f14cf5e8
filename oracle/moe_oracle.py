"""CPU oracle for the quantized Mixture-of-Experts expert path. TEST INFRASTRUCTURE ONLY.

This module is the checker the HIP kernels are compared with. Nothing in the product package imports it;
only the tests, the smoke check and the benchmark's cpu-baseline leg do. It restates, in NumPy alone, the
arithmetic of the reference's own JAX path on a device that has no grouped kernel: dequantize the expert
weights, multiply each expert's sorted rows by its matrix with fp32 sums, SwiGLU with the reference's two
roundings, down projection, fp32-weighted combine. Citations are `file:line` into the reference tree.

What pins each function (tests/test_oracle_golden.py):

* `route`: router_indices (exact) / router_weights (1e-6) of tests/fixtures/moe/{mixtral,deepseek,
  deepseek_v2,deepseek_v4}.npz.
* `sparse_mlp` (fp32 mode): block_output / experts_output of the same files (2e-5).
* `sorted_by_expert`, `sorted_with_shared`: brute force on tiny inputs + invariants (a stable counting sort is a closed form).
* `dequantize_fp8_blocks`: tests/fixtures/codecs/deepseek_kernels.npz `v3/*/dequantized`, bit for bit.
* `decode_mxfp4`: tests/fixtures/gpt_oss/mxfp4.npz `output`, bit for bit.
* `nvfp4_words_to_codes` / `nvfp4_bank_decoded`: the 32 literal encoder masks and the 8-step decode form of
  src/dew/algebra/bits.py:696-705 checked against each other on every basis word and random words; staged
  order known answers of tests/test_gemm_nvfp4.py:37-38; form digest 7fb7f1b609cea47a.
* `combine`: known answer of tests/test_moe_precision.py:652-674 (weights 1/2 +- 2^-11 give 2^-10).
* `relu2` / `expert_mlp(activation='relu2')` (Nemotron-H's ungated experts): that same known answer is stated on a relu2
  layer (up = 1, relu2(1) = 1, down = +-1), which the two-projection path reproduces; the activation itself is the closed
  form max(x, 0)^2 with one rounding, checked on every bf16.
* `expert_mlp(scale_inputs=True)` / `sparse_mlp(scale_inputs=True)` (Llama 4's input-scaled experts, fp32 mode): `output`
  of tests/fixtures/llama4/moe.npz (sigmoid of the top-2 logits on each token's input, the shared expert added) at the
  reference's own tolerance 1e-5 (tests/test_llama4.py:162-191); weighting the outputs instead must miss it by > 1e-3.
* `swiglu`: closed form, the two bf16 roundings checked on hand-computed cases; and every one of the 2048 outputs Torch
  recorded for bf16 `silu(gate) * up` in the reference's tests/fixtures/gated_product/bf16.npz (`swiglu/output`, the
  arm tests/test_causal_transformer.py:1290-1340 holds the reference's product to), bit for bit. `geglu` on the same
  file's `geglu/output`: bit for bit wherever Torch's tanh has not saturated to -1 (there Torch records 0 and the
  reference's logistic form leaves a product below 1e-16).
* `gpt_oss_mlp` (fp32 mode): `output` of tests/fixtures/gpt_oss/moe.npz at the reference's own tolerance (1.6e-4,
  tests/test_gpt_oss.py:45-66): biased router, top-k on the logits, softmax of the chosen, interleaved gate/up
  with both biases, clamp 7, (up + 1) * gate * logistic(1.702 gate). Dropping the down bias must move it by > 0.5.
* `grouped_matmul`: tools/grouped_oracle.py:20-27 semantics (float64 per-group product) on integer inputs,
  where fp32 sums are exact.

* `geglu`: the reference's logistic form of the tanh GELU against the textbook `0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715
  x^3)))` in float64 on every bf16 (a wrong constant, sign or power fails it), and its two roundings on hand cases.
* `silu` / `routed_values` (routed value experts, src/dew/nn/value_experts.py): the reference holds no vectors for the
  layer alone (its fixture is a whole model's logits); `silu` is `swiglu`'s activation with its one rounding, checked
  against `swiglu(x, 1)`, a float64 `x / (1 + e^-x)` and on every bf16; `routed_values` against a token-by-token
  float64 sum of the chosen experts' products on integer operands (where every fp32 sum is exact), which a wrong
  gather, scatter, weight pairing or a missing activation fails.

* `route`'s further switches (`bias_in_weights`, `weight_sum_epsilon`, `weight_sum_min`, `excluded_group_score`,
  `logit_softcap`; src/dew/nn/moe.py:361-384): the reference holds no vectors for them. `excluded_group_score` is pinned
  by the reference's own case restated (tests/test_moe.py:265-292: which experts are chosen, filled at 0.0 and at -inf);
  the others by their definitions in float64 (the biased scores gathered; the sums floored, with the tokens below the
  floor summing to sum / floor and the rest to one; `cap * tanh(x / cap)`, bounded, order-preserving), each of which a
  dropped bias, a floor applied before the epsilon or a cap applied after the scores fails.
* `block_mask` / `route(blocks=, block_experts=)` (LLaDA2.2's block routing): no vectors in the reference; the function is
  the definition's own loops (a block's best selection per expert, its `block_experts` best), checked against a hand case,
  against blocks of one token (where the mask is each token's own top `block_experts`), against one block a row with
  `block_experts = E` (no limit) and against a relabelling of the blocks (which changes nothing).
* `gated_rows` (`shared_gate`, Qwen2-MoE's scalar gate on the shared expert): no vectors in the reference. The dtype flow
  is read from the reference's sources (the gate's Dense under `dtype=bf16`; `logistic`'s one rounding); the arithmetic
  is pinned by a hand case whose three roundings each move the result, and by float64 `sigmoid(x . w) * rows` within bf16.
  `gated_rows_added_f32` (the same gate where the layer states no compute dtype: fp32 throughout, added to the routed rows):
  likewise, by float64 `routed + sigmoid(x . w) * shared` within two fp32 roundings.
* `route(media=, media_bias=)` (DeepSeek-V4.1's image-span bias): by the definition: the media tokens route as a router
  whose bias is `media_bias` routes them, the others as one whose bias is `bias`, row for row.
* `route(given=, covered=)` (replayed routes and the hash router's table rows, `chosen_experts` src/dew/nn/moe.py:202-224):
  no vectors in the reference; pinned by what the definition fixes: the router's own choice given back reproduces its
  weights bit for bit, a permutation of it permutes them, uncovered tokens keep the router's own routing, and the weights
  of arbitrary given experts are the float64 gather-and-normalize of their scores.
* `load_balance_update`: the known answer of tests/test_moe.py:326-336 (counts 3, 1, 0, 0 at rate 0.001).
* `router_statistics`: closed forms (scores = exp(logits - log_z) for softmax; log_z(logits + c) = log_z + c; the
  z-loss's log partition against a float64 logsumexp).
* `rows_quantized` / `blocks_quantized` / `blockwise_fp8_product` (the blockwise FP8 recipe): no byte fixture in
  the reference (its tests hold the product to a float64 truth, tests/test_gemm_blockwise.py:20-40 over
  tests/blockwise_matrix.py); pinned by what the arithmetic fixes: `e4m3_rounded` against a brute-force nearest
  neighbour (ties to the even code) over every fp32 midpoint and grid point of E4M3FN, `power_of_two_ceil` on
  exact powers and their neighbours, the scale rule on amax = 448 * 2^k and on the 1e-4 floor, the quantized
  blocks reproducing tests/fixtures/codecs/deepgemm_fp8.npz's ue8m0 codes and scales wherever the two rules
  agree (they differ only in how amax / 448 is rounded before the ceiling), and the product against the float64
  sum of the dequantized operands at the reference's own bound.

* `mxfp8_quantized` / `mxfp8_product` (the MXFP8 recipe): OCP MX's rule as the reference states it, pinned by its
  invariants (a block's largest magnitude over its scale in [256, 512), so its code is 256 .. 448; 448 .. 512
  saturates; a zero block takes byte 0; the scale byte is the largest magnitude's fp32 exponent field less 8) and
  by the decoded operands reproducing the source within half a code step.

* `nvfp4_quantized` (the NVFP4 recipe's operands): the closed form the reference's own test states
  (tests/test_algebra_bits.py:510-528), checked against the bank quantizer's pins (tests/test_codecs.py) and by
  brute force over the E2M1 grid for the rounding; `nvfp4_block_product` against the float64 sum of the decoded
  operands.

* `kernel_gradient` / `blockwise_fp8_kernel_gradient` and the recipes' `*_gradients` (tests/test_recipe_gradients.py):
  the kernel gradient against the block-by-block definition the reference's own test writes out
  (tests/test_gemm_blockwise.py:97-107, with its shapes, its empty group and scales drawn from [0.5, 2)); both
  gradients of each recipe against the exact derivative (d_x = dy @ w^T, d_w[g] = x_g^T @ dy_g) on operands the format
  holds exactly, where quantizing changes nothing: a wrong axis, transpose, group window or scale pairing fails it.

Parity unpinned (no byte fixture in the reference, closed form only): the exact bits of the softmax
denominator's compensated sum (src/dew/nn/precision.py:1832); it moves router weights by at most one fp32
ulp and no index. `gpt_oss_gating`'s bf16 mode: where each bf16 rounding falls follows JAX's arithmetic on
bf16 arrays (every elementwise operation rounds its result; the logistic is formed in fp32 and rounded once,
src/dew/nn/activations.py:85-98), which no fixture of the reference records in bf16; GPT-OSS's final
`sum(slots * weights)` is restated with fp32 weights and one rounding (`combine`).
"""

import numpy as np

F32 = np.float32

# --------------------------------------------------------------------------------------------------
# Number formats
# --------------------------------------------------------------------------------------------------


def bf16_round(x):
    """fp32 values rounded to bfloat16 (ties to even) and held in fp32: the cast pair the reference's
    `cast_rounded` writes (src/dew/nn/activations.py:281-286). NaN stays NaN."""
    x = np.ascontiguousarray(x, dtype=F32)
    bits = x.view(np.uint32)
    rounded = (bits + (np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1)))) & np.uint32(0xFFFF0000)
    out = rounded.view(F32)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, x, out)
    return out


def bf16_bits(x):
    """The uint16 bit patterns of fp32 values rounded to bfloat16."""
    return (bf16_round(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def bf16_from_bits(bits):
    """fp32 values of bfloat16 bit patterns (uint16)."""
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(F32)


def _e4m3_table():
    """float8_e4m3fn's value for every byte (OCP 8-bit float v1.0: bias 7, no infinities, 0x7f/0xff NaN)."""
    codes = np.arange(256, dtype=np.uint32)
    sign = np.where(codes & 0x80, -1.0, 1.0)
    exponent = ((codes >> 3) & 0xF).astype(np.int32)
    mantissa = (codes & 7).astype(np.float64)
    normal = (1.0 + mantissa / 8.0) * np.exp2(exponent - 7.0)
    subnormal = (mantissa / 8.0) * 2.0 ** -6
    value = np.where(exponent == 0, subnormal, normal) * sign
    value[(codes & 0x7F) == 0x7F] = np.nan
    return value.astype(F32)


E4M3 = _e4m3_table()
"""Value of every float8_e4m3fn byte."""

E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], F32)
"""Value of every E2M1 nibble, sign in bit 3 (src/dew/nn/fake_quant.py:21)."""


# --------------------------------------------------------------------------------------------------
# Dequantizers (the reference dequantizes, then multiplies in the compute dtype)
# --------------------------------------------------------------------------------------------------


def dequantize_fp8_blocks(codes, scale_inv, block=(128, 128)):
    """`f32(code) * scale_inv[i // br, j // bc]` for e4m3 `codes` `[..., rows, cols]` (uint8) and fp32
    `scale_inv` `[..., ceil(rows/br), ceil(cols/bc)]`: src/dew/interop/codecs.py:670-703 (DeepSeek's
    weight-only reading of 128x128 block scales, contract stated at :638-648)."""
    codes = np.asarray(codes, np.uint8)
    rows, cols = codes.shape[-2:]
    br, bc = block
    each = np.repeat(np.repeat(np.asarray(scale_inv, F32), br, axis=-2), bc, axis=-1)[..., :rows, :cols]
    return (E4M3[codes] * each).astype(F32)


def dequantize_fp8_channels(codes, scales):
    """Per-output-channel FP8: `codes [..., depth, width]` e4m3 bytes, `scales [..., width]` fp32, value
    `f32(code) * scale[n]`: the frozen row-scaled rule of src/dew/quantization.py:505-525 (a `(1, K)` block
    on the `[N, K]` view), read back in `[depth, width]` orientation."""
    return (E4M3[np.asarray(codes, np.uint8)] * np.asarray(scales, F32)[..., None, :]).astype(F32)


def decode_mxfp4(blocks, scales):
    """Packed MXFP4 `[expert, out, group, 16]` bytes + E8M0 `[expert, out, group]` bytes to fp32
    `[expert, in, out]`: low nibble first, 32 elements a scale `2^(b-127)`
    (src/dew/interop/codecs.py:115-128,193-224)."""
    blocks = np.asarray(blocks, np.uint8)
    scales = np.asarray(scales, np.uint8)
    experts, outs, groups, _ = blocks.shape
    nibbles = np.stack([blocks & 15, blocks >> 4], axis=-1).reshape(experts, outs, groups, 32)
    power = np.ldexp(F32(1), scales.astype(np.int32) - 127).astype(F32)
    values = E2M1[nibbles] * power[..., None]
    return np.ascontiguousarray(values.reshape(experts, outs, groups * 32).swapaxes(1, 2))


# ---- NVFP4 bank: GF(2)-encoded words in staged depth order ----------------------------------------

NVFP4_ENCODER = (
    0x4000100, 0x8000202, 0x4040401, 0x2800080, 0x1000000, 0x2000000, 0x4000000, 0x8000002,
    0x4040001, 0x20000808, 0x4010000, 0x8020002, 0x4000001, 0x8000000, 0x4040005, 0x20000008,
    0x40001000, 0x80002020, 0x40404010, 0x20080008, 0x10000000, 0x20000000, 0x40000000, 0x80000020,
    0x40400010, 0x2008080, 0x40100000, 0x80200020, 0x40000010, 0x80000000, 0x40400050, 0x2000080)
"""Stored bit i of a word = parity(natural word & NVFP4_ENCODER[i]); the natural word holds code j at bits
4j..4j+3 (src/dew/algebra/bits.py:702-705, `bits.packed` :921-931)."""

NVFP4_MASK = np.uint32(0x81C081C0)
NVFP4_OWED = 256.0
"""The 2^8 the bf16 decode owes the accumulator (src/dew/nn/kernels/formats.py:132-137)."""


def nvfp4_form_digest():
    """The 8-byte version a bank stores beside its words: sha256 of the encoder masks joined by commas,
    first 16 hex digits (src/dew/algebra/bits.py:306-311; src/dew/nn/kernels/formats.py:21)."""
    import hashlib

    return hashlib.sha256(",".join(map(str, NVFP4_ENCODER)).encode()).hexdigest()[:16]


def _rotr32(x, n):
    return (x >> np.uint32(n)) | (x << np.uint32(32 - n))


def nvfp4_words_to_halves(words):
    """The decode form of src/dew/algebra/bits.py:696-700 on stored uint32 words: a rotation by 6, three
    left shifts, four masked xors. Returns uint16 `[..., 8]`: code j's bfloat16 bit pattern, equal to
    `E2M1[code] * 2^-126` (code 2i the low half of register i, 2i+1 the high half)."""
    s = np.asarray(words, np.uint32)
    v1 = _rotr32(s, 6)
    r0 = (s ^ v1) & NVFP4_MASK
    r1 = (s ^ (s << np.uint32(6))) & NVFP4_MASK
    r2 = (s ^ (v1 << np.uint32(2))) & NVFP4_MASK
    r3 = (s << np.uint32(2)) & NVFP4_MASK
    regs = np.stack([r0, r1, r2, r3], axis=-1)
    halves = np.stack([regs & np.uint32(0xFFFF), regs >> np.uint32(16)], axis=-1)
    return halves.reshape(*s.shape, 8).astype(np.uint16)


def nvfp4_words_to_codes(words):
    """Stored words to their eight E2M1 nibbles `[..., 8]` uint8 (sign bit 3), through the decode form: the
    bfloat16 half has the mantissa bit at 6, exponent bits at 7-8 and sign at 15
    (src/dew/algebra/bits.py:683-686)."""
    halves = nvfp4_words_to_halves(words).astype(np.uint32)
    return (((halves >> 6) & 7) | ((halves >> 15) << 3)).astype(np.uint8)


def nvfp4_staged_depths(depth):
    """Depth held by packed row `8w + j` of each 128-deep group: `128 g + 16 j + w`
    (src/dew/nn/kernels/templates/gemm/packed.py:27-33; src/dew/nn/kernels/formats.py:144-155)."""
    if depth % 128:
        raise ValueError(f"an NVFP4 matrix's depth is whole 128-deep groups, not {depth}")
    index = np.arange(depth)
    group, within = np.divmod(index, 128)
    word, code = np.divmod(within, 8)
    return 128 * group + 16 * code + word


def nvfp4_bank_codes(words):
    """A bank's nibbles in natural depth order: `words [E, N, K/8]` uint32 to uint8 `[E, K, N]`."""
    words = np.asarray(words, np.uint32)
    experts, width, nwords = words.shape
    staged = nvfp4_words_to_codes(words).reshape(experts, width, nwords * 8)   # staged position p = 8w + j
    natural = np.empty_like(staged)
    natural[..., nvfp4_staged_depths(nwords * 8)] = staged
    return np.ascontiguousarray(natural.swapaxes(1, 2))


def nvfp4_bank_decoded(words, scales):
    """`NvFp4.decoded()` (src/dew/nn/kernels/formats.py:108-113): each code times its 16-block's e4m3 scale
    over 2^8, exactly representable in bfloat16, `[E, K, N]` fp32. `scales [E, N, K/16]` are e4m3 bytes."""
    codes = nvfp4_bank_codes(words)
    owed = (E4M3[np.asarray(scales, np.uint8)] * F32(1.0 / NVFP4_OWED)).swapaxes(1, 2)      # [E, K/16, N]
    values = E2M1[codes] * np.repeat(owed, 16, axis=1)
    rounded = bf16_round(values)
    assert np.array_equal(rounded, values), "an NVFP4 value over 2^8 is exact in bfloat16"
    return rounded


def nvfp4_bank_factor(scale):
    """`NvFp4.factor`: 2^8 times each expert's tensor scale (src/dew/nn/kernels/formats.py:132-137)."""
    return (F32(NVFP4_OWED) * np.asarray(scale, F32)).astype(F32)


# --------------------------------------------------------------------------------------------------
# Router (src/dew/nn/moe.py:466-565)
# --------------------------------------------------------------------------------------------------

_LN2_HI, _LN2_LO = F32(0.693145751953125), F32(1.428606765330187e-06)
_EXP_TERMS = tuple(F32(t) for t in (1.0 / 5040.0, 1.0 / 720.0, 1.0 / 120.0, 1.0 / 24.0, 1.0 / 6.0, 0.5, 1.0, 1.0))
_INV_LN2 = F32(1.0 / np.log(2.0))


def exp_f32(x):
    """`e^x` in fp32 by one fixed sequence of IEEE fp32 operations, no fused multiply-add: Cody-Waite
    reduction `x = n ln2 + r`, Taylor sum to r^7 by Horner, times 2^n in two exact steps. The algorithm is
    the reference's own portable exp (src/dew/nn/precision.py:470-488); the HIP router runs the same
    sequence, so scores and hence top-k choices agree bit for bit between the two."""
    x = np.clip(np.asarray(x, F32), F32(-104.0), F32(90.0))
    n = np.rint(x * _INV_LN2).astype(F32)
    r = ((x - n * _LN2_HI).astype(F32) - (n * _LN2_LO).astype(F32)).astype(F32)
    p = np.full_like(r, _EXP_TERMS[0])
    for term in _EXP_TERMS[1:]:
        p = ((p * r).astype(F32) + term).astype(F32)
    n = n.astype(np.int32)
    half = n // 2                                  # floor division: both halves stay normal exponents
    first = np.ldexp(F32(1), half).astype(F32)
    second = np.ldexp(F32(1), n - half).astype(F32)
    return ((p * first).astype(F32) * second).astype(F32)


def _sum_rounded_once(values):
    """Sum over the last axis, rounded once to fp32: the role of `compensated_sum`
    (src/dew/nn/precision.py:1832-1844). Realised as a float64 sum in one fixed order (64 interleaved
    partial sums, then a halving tree), the order the HIP router's wave reduction uses."""
    v = np.asarray(values, np.float64)
    count = v.shape[-1]
    lanes = np.zeros((*v.shape[:-1], 64), np.float64)
    for start in range(0, count, 64):
        chunk = v[..., start:start + 64]
        lanes[..., :chunk.shape[-1]] += chunk
    width = 32
    while width >= 1:
        lanes = lanes[..., :width] + lanes[..., width:2 * width]
        width //= 2
    return lanes[..., 0].astype(F32)


def expert_softmax(logits):
    """src/dew/nn/moe.py:184-191: exp(x - max) over their once-rounded sum, IEEE division."""
    logits = np.asarray(logits, F32)
    shifted = exp_f32(logits - logits.max(axis=-1, keepdims=True))
    return (shifted / _sum_rounded_once(shifted)[..., None]).astype(F32)


def logistic(x, exp=exp_f32):
    """`1 / (1 + e^-x)` in fp32 with a true division (src/dew/nn/precision.py:568-575)."""
    x = np.asarray(x, F32)
    return (F32(1) / (F32(1) + exp(-x)).astype(F32)).astype(F32)


def sqrt_softplus(x):
    """DeepSeek V4's score `sqrt(softplus(x))` (src/dew/nn/moe.py:539-540); float64 inside, for the
    fixture's sake only (no BASELINE config uses it)."""
    x = np.asarray(x, np.float64)
    return np.sqrt(np.logaddexp(0.0, x)).astype(F32)


def top_k(values, k):
    """`jax.lax.top_k`: the k largest along the last axis in descending order, ties to the lower index.
    Returns (values, indices int32)."""
    values = np.asarray(values)
    order = np.argsort(-values, axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(values, order, axis=-1), order.astype(np.int32)


def capped_logits(logits, softcap):
    """`capped_logits` (src/dew/nn/precision.py:2086-2092) as the router applies it (src/dew/nn/moe.py:526-534):
    `cap * tanh(logits / cap)` in fp32, the logits themselves where there is no cap."""
    logits = np.asarray(logits, F32)
    if softcap is None:
        return logits
    cap = F32(softcap)
    return (cap * np.tanh((logits / cap).astype(F32)).astype(F32)).astype(F32)


def block_mask(selection, blocks, experts):
    """`Router.block_mask` (src/dew/nn/moe.py:566-585): True where an expert is one of the `experts` best of its token's
    block, a block's score for an expert its best token's selection; `selection [rows, length, E]`, `blocks [rows, length]`
    numbering each row's blocks from 0, a negative id (padding) a block of its own. Written as the definition's loops."""
    selection, blocks = np.asarray(selection, F32), np.asarray(blocks)
    kept = np.zeros(selection.shape, bool)
    for row in range(selection.shape[0]):
        ids = np.where(blocks[row] < 0, -1, blocks[row])
        for block in np.unique(ids):
            members = np.flatnonzero(ids == block)
            best = selection[row, members].max(axis=0)
            _, allowed = top_k(best, experts)
            kept[np.ix_([row], members, allowed)] = True
    return kept


def selection_scores(logits, *, score_function="softmax", bias=None, expert_groups=1, groups_per_token=1, group_score="top2",
                     excluded_group_score=None, media=None, media_bias=None, blocks=None, block_experts=None):
    """(scores, selection) of `Router.__call__` (src/dew/nn/moe.py:466-470, 516-524): the activated scores and what the
    top-k runs over, the scores plus the bias with the experts outside a token's best groups at -inf, or at
    `excluded_group_score` where the router fills one in (:496-565)."""
    logits = np.asarray(logits, F32)
    experts = logits.shape[-1]
    if score_function == "softmax":
        scores = expert_softmax(logits)
    elif score_function == "sigmoid":
        scores = logistic(logits)
    elif score_function == "sqrtsoftplus":
        scores = sqrt_softplus(logits)
    else:
        raise ValueError(score_function)
    selection = scores if bias is None else (scores + np.asarray(bias, F32)).astype(F32)
    if media is not None:      # a media token's own bias (`selection`, src/dew/nn/moe.py:516-524)
        selection = np.where(np.asarray(media, bool)[..., None], (scores + np.asarray(media_bias, F32)).astype(F32), selection)
    if blocks is not None:     # outside each block's shortlist -inf (`selection`, src/dew/nn/moe.py:522-523)
        selection = np.where(block_mask(np.where(np.isnan(selection), F32(-np.inf), selection), blocks, block_experts), selection, F32(-np.inf))
    # A NaN selection competes as -inf (the HIP router's rule): none of the reference's tests feeds its `lax.top_k` a
    # NaN, so this is a choice of this restatement, made so that every choice stays an expert in range.
    selection = np.where(np.isnan(selection), F32(-np.inf), selection)
    if expert_groups > 1:
        per_group = experts // expert_groups
        grouped = selection.reshape(*selection.shape[:-1], expert_groups, per_group)
        if group_score == "max":
            group_scores = grouped.max(axis=-1)
        else:
            best_two, _ = top_k(grouped, 2)
            group_scores = (best_two[..., 0] + best_two[..., 1]).astype(F32)
        _, groups = top_k(group_scores, groups_per_token)
        kept = np.zeros(group_scores.shape, bool)
        np.put_along_axis(kept, groups, True, axis=-1)
        fill = F32(-np.inf) if excluded_group_score is None else F32(excluded_group_score)
        selection = np.where(np.repeat(kept, per_group, axis=-1), selection, fill)
    return scores, selection


def top_k_margin(selection, top_k_count):
    """The least gap, over the tokens, between the last selection chosen and the best one left out, as (gap, the gap in
    units of the chosen value's fp32 spacing, token). A gap of zero is a tie, which the lower index wins in every
    implementation; a gap of a few spacings is where two exponentials that round differently could choose differently."""
    selection = np.asarray(selection, F32)
    if selection.shape[-1] <= top_k_count:
        return float("inf"), float("inf"), -1
    ranked = -np.sort(-selection.reshape(-1, selection.shape[-1]), axis=-1)
    last, left = ranked[:, top_k_count - 1], ranked[:, top_k_count]
    gap = (last.astype(np.float64) - left.astype(np.float64))
    gap[~np.isfinite(left)] = np.inf
    token = int(gap.argmin())
    return float(gap[token]), float(gap[token] / np.spacing(np.abs(last[token]))), token


def route(logits, top_k_count, *, score_function="softmax", normalize_weights=True, bias=None,
          routed_scaling_factor=1.0, expert_groups=1, groups_per_token=1, group_score="top2",
          weight_sum_epsilon=1e-20, weight_sum_min=0.0, bias_in_weights=False, excluded_group_score=None,
          logit_softcap=None, given=None, covered=None, media=None, media_bias=None, blocks=None, block_experts=None):
    """`Router.__call__` from its logits on (src/dew/nn/moe.py:466-494): the cap on the logits (:526-534), scores,
    selection (bias, group-limited mask :496-565), top-k, weights (:483-494: a softmax router renormalizes the chosen
    logits unless `bias_in_weights` or `weight_sum_min` say otherwise; else the chosen scores, plus the bias under
    `bias_in_weights`, over `max(sum + weight_sum_epsilon, weight_sum_min)`). `given` [T, k] are experts used in place
    of the top-k for the tokens `covered` [T] marks (all where None). Returns (weights fp32 [T, k], indices int32 [T, k])."""
    logits = capped_logits(logits, logit_softcap)
    scores, selection = selection_scores(logits, score_function=score_function, bias=bias, expert_groups=expert_groups,
                                         groups_per_token=groups_per_token, group_score=group_score,
                                         excluded_group_score=excluded_group_score, media=media, media_bias=media_bias,
                                         blocks=blocks, block_experts=block_experts)
    _, indices = top_k(selection, top_k_count)
    valid = None
    if given is not None:      # `chosen_experts` (src/dew/nn/moe.py:202-224): a replayed record, or the hash table's rows (:500-507)
        given = np.asarray(given).astype(np.int32)
        indices = given if covered is None else np.where(np.asarray(covered, bool)[..., None], given, indices).astype(np.int32)
        # ids outside the experts (a dropped slot's sentinel) pass through as they are; such a slot weighs nothing and takes
        # no part in the other slots' normalization (the sort drops it, src/dew/nn/moe.py:1101-1128)
        valid = (indices >= 0) & (indices < logits.shape[-1])
        if valid.all():
            valid = None
    safe = indices if valid is None else np.clip(indices, 0, logits.shape[-1] - 1)
    if normalize_weights and score_function == "softmax" and not bias_in_weights and not weight_sum_min:
        if valid is None:
            weights = expert_softmax(np.take_along_axis(logits, safe, axis=-1))        # moe.py:194-199,485
        else:
            chosen = np.where(valid, np.take_along_axis(logits, safe, axis=-1), F32(-np.inf)).astype(F32)
            with np.errstate(invalid="ignore", divide="ignore"):
                shifted = np.where(valid, exp_f32(np.where(valid, chosen - chosen.max(axis=-1, keepdims=True), F32(0))), F32(0)).astype(F32)
                weights = (shifted / _sum_rounded_once(shifted)[..., None]).astype(F32)
    else:
        gating = (scores + np.asarray(bias, F32)).astype(F32) if bias_in_weights else scores
        weights = np.take_along_axis(gating, safe, axis=-1)
        if valid is not None:
            weights = np.where(valid, weights, F32(0)).astype(F32)
        if normalize_weights:
            total = weights[..., 0].copy()
            for j in range(1, top_k_count):
                total = (total + weights[..., j]).astype(F32)
            total = (total + F32(weight_sum_epsilon)).astype(F32)
            if weight_sum_min:
                total = np.maximum(total, F32(weight_sum_min))
            weights = (weights / total[..., None]).astype(F32)
    if valid is not None:
        weights = np.where(valid, weights, F32(0)).astype(F32)
    return (weights * F32(routed_scaling_factor)).astype(F32), indices


def router_statistics(logits, *, score_function="softmax"):
    """What the router sows beside its choices (src/dew/nn/moe.py:474-479): the activated scores `[T, E]`
    (`_activated`, :536-541) and the log partition of the logits `[T]`, `jax.nn.logsumexp`'s max + log(sum(exp(x -
    max))) in fp32."""
    logits = np.asarray(logits, F32)
    scores = expert_softmax(logits) if score_function == "softmax" else logistic(logits)
    top = logits.max(axis=-1, keepdims=True)
    log_z = (top[..., 0] + np.log(np.exp((logits - top).astype(np.float64)).sum(axis=-1)).astype(F32)).astype(F32)
    return scores, log_z


def load_balance_update(counts, rate):
    """src/dew/nn/moe.py:271-300, the integer branch: direction -1 where a count is above floor(sum / E), +1 where
    below it or (at it) the sum leaves a remainder, else 0; times `rate` in fp32."""
    counts = np.asarray(counts, np.int64)
    average, remainder = divmod(int(counts.sum()), counts.size)
    direction = np.where(counts > average, -1, np.where((counts < average) | (remainder > 0), 1, 0))
    return (F32(rate) * direction.astype(F32)).astype(F32)


def router_logits(x, kernel):
    """`Router.logits` (src/dew/nn/moe.py:526-534): IEEE fp32 product of the tokens (widened to fp32) and
    the `[D, E]` fp32 kernel."""
    return (np.asarray(x, F32) @ np.asarray(kernel, F32)).astype(F32)


# --------------------------------------------------------------------------------------------------
# Dispatch (src/dew/nn/moe.py:1101-1128)
# --------------------------------------------------------------------------------------------------


def sorted_by_expert(indices, num_experts):
    """`_sorted_locally`'s bookkeeping: stable argsort of the flattened expert ids, group sizes, offsets,
    and the token row each sorted slot reads. Returns dict(order, rows, sizes, offsets), all int32."""
    indices = np.asarray(indices)
    k = indices.shape[-1]
    experts = indices.reshape(-1)
    order = np.argsort(experts, kind="stable").astype(np.int32)
    sizes = np.bincount(experts, minlength=num_experts)[:num_experts].astype(np.int32)
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    return {"order": order, "rows": (order // k).astype(np.int32), "sizes": sizes, "offsets": offsets}


def sorted_with_shared(indices, num_experts, shared_rows):
    """`sorted_by_expert` with an always-on expert as group `num_experts`: behind the routed slots come `shared_rows`
    more slots of that group, slot `R + i` reading token i (src/dew/nn/moe.py:1497-1503 runs that expert as a dense MLP
    over every token; as one more group of the sort its rows ride the routed experts' launches). Dropped slots (an id
    outside [0, num_experts)) sort behind it. Returns dict(order, rows, sizes [E + 1], offsets [E + 2])."""
    indices = np.asarray(indices)
    k = indices.shape[-1]
    routed = indices.size
    ids = indices.reshape(-1).astype(np.int64)
    ids = np.where((ids < 0) | (ids >= num_experts), num_experts + 1, ids)
    buckets = np.concatenate([ids, np.full(shared_rows, num_experts, np.int64)])
    order = np.argsort(buckets, kind="stable").astype(np.int32)
    sizes = np.bincount(buckets, minlength=num_experts + 1)[:num_experts + 1].astype(np.int32)
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    rows = np.where(order < routed, order // k, order - routed).astype(np.int32)
    return {"order": order, "rows": rows, "sizes": sizes, "offsets": offsets}


# --------------------------------------------------------------------------------------------------
# Grouped products, SwiGLU, combine
# --------------------------------------------------------------------------------------------------


def grouped_matmul(x, w, sizes, *, dtype="bfloat16", factor=None, accumulate=F32):
    """Each group's leading rows of `x [rows, depth]` times its matrix `w [groups, depth, width]`
    (`jax.lax.ragged_dot` semantics, src/dew/nn/kernels/xla_products.py:86-115): operands rounded to the
    compute dtype, products summed in fp32 (`accumulate`), one rounding to the compute dtype; rows past
    `sum(sizes)` are zero. `factor [groups]` multiplies the fp32 sums before the rounding (the NVFP4
    bank's deferred factor, src/dew/nn/kernels/gemm.py:660-662)."""
    x = np.asarray(x, F32)
    w = np.asarray(w, F32)
    if dtype == "bfloat16":
        x = bf16_round(x)
    out = np.zeros((x.shape[0], w.shape[2]), F32)
    start = 0
    for group, size in enumerate(np.asarray(sizes).tolist()):
        if size:
            matrix = bf16_round(w[group]) if dtype == "bfloat16" else w[group]
            summed = (x[start:start + size].astype(accumulate) @ matrix.astype(accumulate))
            if factor is not None:
                summed = summed.astype(F32) * F32(factor[group])
            out[start:start + size] = summed.astype(F32)
        start += size
    return bf16_round(out) if dtype == "bfloat16" else out


# --------------------------------------------------------------------------------------------------
# The blockwise FP8 recipe's forward product (activations quantized 1 x 128, weights 128 x 128)
# --------------------------------------------------------------------------------------------------

SCALE_DEPTH = 128
E4M3_MAX = F32(448.0)


def power_of_two_ceil(value):
    """The least power of two >= `value` read off its fp32 bits: its exponent, plus one where any fraction
    bit is set (src/dew/nn/fake_quant.py:48-57; normal values only, which a floored amax / 448 always is)."""
    bits = np.ascontiguousarray(value, F32).view(np.uint32)
    field = (bits >> np.uint32(23)) & np.uint32(0xFF)
    field = field + ((bits & np.uint32(0x7FFFFF)) != 0)
    return (field.astype(np.uint32) << np.uint32(23)).view(F32)


def e4m3_rounded(values):
    """fp32 values within +-448 rounded to E4M3FN, ties to even, by arithmetic (src/dew/nn/fake_quant.py:60-76):
    the quantum is 2^(max(exponent, -6) - 3); the quotient by it is exact and `rint` ties to the even multiple."""
    values = np.ascontiguousarray(values, F32)
    exponent = ((values.view(np.uint32) >> np.uint32(23)) & np.uint32(0xFF)).astype(np.int32) - 127
    quantum = np.exp2(np.maximum(exponent, -6) - 3).astype(F32)
    return (np.rint(values / quantum) * quantum).astype(F32)


def e4m3_bytes(values):
    """The float8_e4m3fn byte of each value already on the E4M3FN grid (the `.astype(float8_e4m3fn)` of an exact
    value; -0.0 keeps its sign)."""
    values = np.ascontiguousarray(values, F32)
    magnitudes = E4M3[:0x7F].astype(F32)  # ascending, 0 .. 448
    index = np.searchsorted(magnitudes, np.abs(values))
    assert np.array_equal(magnitudes[index], np.abs(values)), "a value off the E4M3FN grid"
    return (index | np.where(np.signbit(values), 0x80, 0)).astype(np.uint8)


def fp8_scaled_blocks(x, block):
    """`x` in fp32 blocks of `block` channels and each block's power-of-two scale: amax floored at 1e-4, the scale
    the ceiling power of two of amax * f32(1 / 448) (src/dew/nn/fake_quant.py:117-122)."""
    blocks = np.asarray(x, F32).reshape(*np.shape(x)[:-1], -1, block)
    amax = np.maximum(np.abs(blocks).max(axis=-1, keepdims=True), F32(1e-4)).astype(F32)
    return blocks, power_of_two_ceil(amax * F32(1 / 448.0))


def fp8_codes(values):
    """src/dew/nn/fake_quant.py:125-128: clamp to +-448, round to E4M3FN."""
    return e4m3_rounded(np.clip(np.asarray(values, F32), -E4M3_MAX, E4M3_MAX))


def rows_quantized(x):
    """`x [..., n]` as E4M3 values a 1 x 128 tile at a time along its last axis and each tile's power-of-two scale
    `[..., n / 128]` (src/dew/nn/kernels/projections.py:176-182). Returns (values on the E4M3 grid, scales)."""
    blocks, scale = fp8_scaled_blocks(x, SCALE_DEPTH)
    return fp8_codes(blocks / scale).reshape(np.shape(x)), scale[..., 0]


def blocks_quantized(w):
    """`w [groups, depth, width]` as E4M3 values a 128 x 128 block at a time and each block's power-of-two scale
    `[groups, depth / 128, width / 128]` (src/dew/nn/kernels/projections.py:185-196)."""
    w = np.asarray(w, F32)
    groups, depth, width = w.shape
    edge = SCALE_DEPTH
    tiled = w.reshape(groups, depth // edge, edge, width // edge, edge).transpose(0, 1, 3, 2, 4)
    blocks, scale = fp8_scaled_blocks(tiled.reshape(groups, depth // edge, width // edge, -1), edge * edge)
    codes = fp8_codes(blocks / scale).reshape(tiled.shape).transpose(0, 1, 3, 2, 4)
    return codes.reshape(w.shape), scale[..., 0, 0]


def twice_scaled(product, first, second):
    """`product` times two scales in the order whose intermediate is a normal fp32
    (src/dew/nn/precision.py:1782-1791)."""
    product, first, second = np.broadcast_arrays(np.asarray(product, F32), np.asarray(first, F32), np.asarray(second, F32))
    tiny = np.finfo(F32).tiny
    with np.errstate(over="ignore", under="ignore"):
        once = (product * first).astype(F32)
        kept = np.isfinite(once) & ((np.abs(once) >= tiny) | (product == 0))
        return (np.where(kept, once, (product * second).astype(F32)) * np.where(kept, second, first)).astype(F32)


def blockwise_fp8_product(lhs, kernel, group_sizes, row_scales, column_scales, *, dtype="bfloat16", bias=None):
    """Each group's rows of `lhs [rows, depth]` (E4M3 values) times its matrix of `kernel [groups, depth, width]`
    (E4M3 values), each 128-deep block's partial, summed exactly and rounded to fp32, times its rows' scales
    (`row_scales [depth / 128, rows]`) and its group's column scales (`column_scales [groups, depth / 128, width / c]`)
    before it is added, in the blocks' order, into the fp32 sum; one rounding to `dtype`; rows past the groups are
    zero (src/dew/nn/kernels/gemm.py:764-793 over src/dew/nn/kernels/xla_products.py:147-173). `bias [groups,
    width]` is added to the fp32 sums before the rounding (src/dew/nn/kernels/projections.py:107-140).
    The partial of 128 products of 8-bit-mantissa values is exact in float64."""
    lhs, kernel = np.asarray(lhs, F32), np.asarray(kernel, F32)
    row_scales, column_scales = np.asarray(row_scales, F32), np.asarray(column_scales, F32)
    blocks, rows = row_scales.shape
    groups, _, scaled = column_scales.shape
    width = kernel.shape[2]
    assert lhs.shape == (rows, blocks * SCALE_DEPTH) and kernel.shape[:2] == (groups, blocks * SCALE_DEPTH) and width % scaled == 0
    total = np.zeros((rows, width), F32)
    start = 0
    for group, size in enumerate(np.asarray(group_sizes).tolist()):
        span = slice(start, start + size)
        for index in range(blocks if size else 0):
            depth = slice(index * SCALE_DEPTH, (index + 1) * SCALE_DEPTH)
            partial = (lhs[span, depth].astype(np.float64) @ kernel[group, depth].astype(np.float64)).astype(F32)
            columns = np.repeat(column_scales[group, index], width // scaled)[None, :]
            total[span] = total[span] + twice_scaled(partial, row_scales[index, span, None], columns)
        if bias is not None and size:
            total[span] = total[span] + np.asarray(bias, F32)[group][None, :]
        start += size
    return bf16_round(total) if dtype == "bfloat16" else total


def blockwise_fp8_projection(x, w, group_sizes, *, dtype="bfloat16", bias=None):
    """Each group's rows of `x` times its matrix of `w` in the blockwise FP8 recipe: both quantized
    (`rows_quantized`, `blocks_quantized`), their product `blockwise_fp8_product`
    (src/dew/nn/kernels/projections.py:199-204; with ragged groups and a bias, `recipe_projection` :96-140, whose
    zero padding rows add nothing)."""
    rows, rows_scales = rows_quantized(x)
    blocks, blocks_scales = blocks_quantized(w)
    return blockwise_fp8_product(rows, blocks, group_sizes, rows_scales.T, blocks_scales, dtype=dtype, bias=bias)


# --------------------------------------------------------------------------------------------------
# The MXFP8 recipe's forward product (OCP MX: E4M3 codes, a power-of-two E8M0 scale every 32 depths)
# --------------------------------------------------------------------------------------------------

MX_DEPTH = 32


def mxfp8_quantized(x):
    """`x [..., depth]` as MXFP8 by OCP MX's rule (src/dew/nn/kernels/formats.py:195-229): each 32 depths' scale 2
    to the power of its largest magnitude's binary exponent less 8, so that the magnitude over the scale lies in
    [256, 512); each value over its scale rounded to E4M3, ties to even, saturating at +-448; a block of zeros
    takes the least scale 2^-127; exponents clipped to +-127. Returns (E4M3 values `[..., depth]`, E8M0 bytes
    `[..., depth / 32]`: scale = 2^(byte - 127))."""
    x = np.asarray(x, F32)
    blocks = x.reshape(*x.shape[:-1], x.shape[-1] // MX_DEPTH, MX_DEPTH)
    largest = np.abs(blocks).max(axis=-1, keepdims=True)
    binade = np.frexp(largest)[1]
    exponent = np.clip(np.where(largest > 0, binade - 1 - 8, -127), -127, 127).astype(np.int32)
    scaled = np.ldexp(blocks.astype(np.float64), -exponent).astype(F32)  # exact: a power of two, within fp32's range
    return fp8_codes(scaled).reshape(x.shape), (exponent[..., 0] + 127).astype(np.uint8)


def mxfp8_decoded(values, scales):
    """src/dew/nn/kernels/formats.py:231-243: each E4M3 value times its block's scale 2^(byte - 127), in float64
    (exact)."""
    exponents = np.repeat(np.asarray(scales).astype(np.int32) - 127, MX_DEPTH, axis=-1)
    return np.ldexp(np.asarray(values, np.float64), exponents)


def mxfp8_product(lhs, lhs_scales, matrices, matrix_scales, group_sizes, *, dtype="bfloat16", bias=None):
    """Each group's rows of `lhs [rows, depth]` times its matrix of `matrices [groups, width, depth]` (K-major), both
    MXFP8: each value its code times its 32 depths' scale, every product exact, summed in fp32 and rounded once
    (src/dew/nn/kernels/gemm.py:882-892); rows past the groups zero. The sum is formed exactly (float64) and
    rounded to fp32, which any order of fp32 additions reaches to a few ulps."""
    left = mxfp8_decoded(lhs, lhs_scales)
    right = mxfp8_decoded(matrices, matrix_scales)
    rows, width = left.shape[0], right.shape[1]
    total = np.zeros((rows, width), F32)
    start = 0
    for group, size in enumerate(np.asarray(group_sizes).tolist()):
        if size:
            summed = (left[start:start + size] @ right[group].T).astype(F32)
            if bias is not None:
                summed = summed + np.asarray(bias, F32)[group][None, :]
            total[start:start + size] = summed
        start += size
    return bf16_round(total) if dtype == "bfloat16" else total


def mxfp8_projection(x, w, group_sizes, *, dtype="bfloat16", bias=None):
    """`x [rows, depth]` and `w [groups, depth, width]` both quantized along the depth, their `mxfp8_product`
    (src/dew/nn/kernels/projections.py:231-258)."""
    rows, row_scales = mxfp8_quantized(x)
    matrices, matrix_scales = mxfp8_quantized(np.swapaxes(np.asarray(w, F32), 1, 2))
    return mxfp8_product(rows, row_scales, matrices, matrix_scales, group_sizes, dtype=dtype, bias=bias)


# --------------------------------------------------------------------------------------------------
# The recipes' gradients: the input's is the recipe's own product of the requantized cotangent and the matrices
# quantized along the width; the matrices' contracts each group's tokens
# --------------------------------------------------------------------------------------------------


def kernel_gradient(lhs_t, rhs_t, group_sizes, *, dtype="bfloat16"):
    """Each group's tokens contracted: `out[g] = lhs_t[:, tokens of g] @ rhs_t[:, tokens of g].T` for operands
    `[depth, tokens]` and `[width, tokens]` already decoded to their values (float64, exact), summed exactly, rounded to
    fp32 and then to `dtype`; an empty group's is zero (`gemm_t`, src/dew/nn/kernels/gemm.py:418-431; the definition the
    reference's own test writes out, tests/test_gemm_blockwise.py:97-107)."""
    lhs_t, rhs_t = np.asarray(lhs_t, np.float64), np.asarray(rhs_t, np.float64)
    out = np.zeros((len(group_sizes), lhs_t.shape[0], rhs_t.shape[0]), F32)
    start = 0
    for group, size in enumerate(np.asarray(group_sizes, np.int64)):
        out[group] = (lhs_t[:, start:start + size] @ rhs_t[:, start:start + size].T).astype(F32)
        start += size
    return bf16_round(out) if dtype == "bfloat16" else out


def blockwise_fp8_kernel_gradient(lhs_t, rhs_t, group_blocks, row_scales, column_scales, *, dtype="bfloat16"):
    """src/dew/nn/kernels/gemm.py:795-819: E4M3 values `lhs_t [depth, rows]` and `rhs_t [width, rows]`, each 128-row
    block's partial times its depth rows' scales (`row_scales [rows / 128, depth]`) and its columns'
    (`column_scales [rows / 128, width]`), added into its group's sum."""
    left = np.asarray(lhs_t, np.float64) * np.repeat(np.asarray(row_scales, np.float64).T, SCALE_DEPTH, axis=1)
    right = np.asarray(rhs_t, np.float64) * np.repeat(np.asarray(column_scales, np.float64).T, SCALE_DEPTH, axis=1)
    return kernel_gradient(left, right, np.asarray(group_blocks) * SCALE_DEPTH, dtype=dtype)


def blockwise_fp8_gradients(x, w, cotangent, group_blocks, *, dtype="bfloat16"):
    """`_projection_backward` (src/dew/nn/kernels/projections.py:211-224): the input's gradient is the recipe's product
    of the cotangent, requantized along the width, and the matrices' blocks transposed; the matrices' is the kernel
    gradient of `x.T` and `cotangent.T`, each quantized along the tokens. Returns (d_x, d_w)."""
    sizes = np.asarray(group_blocks) * SCALE_DEPTH
    dy, dy_scales = rows_quantized(cotangent)
    blocks, blocks_scales = blocks_quantized(w)
    d_x = blockwise_fp8_product(dy, np.swapaxes(blocks, 1, 2), sizes, dy_scales.T, np.swapaxes(blocks_scales, 1, 2), dtype=dtype)
    rows_t, rows_t_scales = rows_quantized(np.asarray(x, F32).T)
    dy_t, dy_t_scales = rows_quantized(np.asarray(cotangent, F32).T)
    return d_x, blockwise_fp8_kernel_gradient(rows_t, dy_t, group_blocks, rows_t_scales.T, dy_t_scales.T, dtype=dtype)


def mxfp8_gradients(x, w, cotangent, group_blocks, *, dtype="bfloat16"):
    """`_mx_backward` (src/dew/nn/kernels/projections.py:263-275): d_x = the MXFP8 product of the cotangent and the
    matrices both quantized along the width; d_w = each group's tokens contracted over `x.T` and `cotangent.T`
    quantized along the tokens, every 32 a scale, and decoded (exact in bf16), fp32 sums. Returns (d_x, d_w)."""
    sizes = np.asarray(group_blocks) * SCALE_DEPTH
    d_x = mxfp8_product(*mxfp8_quantized(cotangent), *mxfp8_quantized(np.asarray(w, F32)), sizes, dtype=dtype)
    rows_t = mxfp8_decoded(*mxfp8_quantized(np.asarray(x, F32).T))
    dy_t = mxfp8_decoded(*mxfp8_quantized(np.asarray(cotangent, F32).T))
    return d_x, kernel_gradient(rows_t, dy_t, sizes, dtype=dtype)


def nvfp4_gradients(x, w, cotangent, group_blocks, *, dtype="bfloat16"):
    """`_nvfp4_backward` (src/dew/nn/kernels/projections.py:322-337): d_x = the NVFP4 block product of the cotangent and
    the matrices both quantized along the width; d_w = each group's tokens contracted over `x.T` and `cotangent.T`
    quantized along the tokens (every 16 a scale) and decoded with their tensor scales, summed at the highest precision.
    Returns (d_x, d_w). (`nvfp4_quantized` and `nvfp4_projection` are defined below.)"""
    sizes = np.asarray(group_blocks) * SCALE_DEPTH
    d_x = nvfp4_projection(cotangent, np.swapaxes(np.asarray(w, F32), 1, 2), sizes, dtype=dtype)
    decoded = []
    for operand in (x, cotangent):
        values, scales, tensor = nvfp4_quantized(np.asarray(operand, F32).T)
        decoded.append(values.astype(np.float64) * np.repeat(scales.astype(np.float64), 16, axis=1) * np.float64(tensor))
    return d_x, kernel_gradient(decoded[0], decoded[1], sizes, dtype=dtype)


# --------------------------------------------------------------------------------------------------
# The NVFP4 recipe's forward product (E2M1 codes, an E4M3 scale every 16 depths, one tensor scale)
# --------------------------------------------------------------------------------------------------


def nvfp4_quantized(x):
    """`x [..., depth]` as NVFP4 along its depth (`NvFp4Block.quantized`, src/dew/nn/kernels/formats.py:263-274, over
    `bits.nvfp4_coded`, src/dew/algebra/bits.py:941-982, in the closed form its test states,
    tests/test_algebra_bits.py:510-528): one tensor scale, the largest magnitude over 6 x 448 (fp32's least normal
    at least; 1 for a zero tensor); each 16 depths' scale the least E4M3 at or above its largest magnitude over the
    tensor scale over 6; each value, divided by the tensor scale and then by its block's, rounded to E2M1, ties to
    even; a zero block's codes zero. Every quotient an IEEE fp32 division. Returns (E2M1 values `[..., depth]`, E4M3
    scale values `[..., depth / 16]`, the tensor scale)."""
    x = np.asarray(x, F32)
    largest = F32(np.abs(x).max()) if x.size else F32(0)
    tensor = np.maximum(largest / F32(6 * 448), np.finfo(F32).tiny).astype(F32) if largest > 0 else F32(1)
    blocks = np.abs(x).reshape(*x.shape[:-1], x.shape[-1] // 16, 16)
    ratio = ((blocks.max(axis=-1) / tensor).astype(F32) / F32(6)).astype(F32)
    table = E4M3[:0x7F].astype(F32)
    scales = table[np.minimum(np.searchsorted(table, ratio), table.size - 1)]
    each = np.repeat(scales, 16, axis=-1)
    positive = each > 0
    quotient = np.where(positive, ((x / tensor).astype(F32) / np.where(positive, each, F32(1))).astype(F32), F32(0))
    grid = E2M1[:8].astype(np.float64)
    magnitude = np.abs(quotient.astype(np.float64))
    below = np.searchsorted((grid[1:] + grid[:-1]) / 2, magnitude, side="left")    # a tie stays with the lower code
    above = np.searchsorted((grid[1:] + grid[:-1]) / 2, magnitude, side="right")   # a tie goes to the upper code
    code = np.where((above != below) & (above % 2 == 1), below, above)             # ... whichever is even
    return (np.copysign(grid[code], quotient)).astype(F32), scales, tensor


def nvfp4_block_product(lhs, lhs_scales, lhs_scale, matrices, matrix_scales, matrix_scale, group_sizes, *, dtype="bfloat16", bias=None):
    """Each group's rows of `lhs [rows, depth]` times its matrix of `matrices [groups, width, depth]`, both NVFP4:
    each code times its sixteen depths' scale, every product exact, summed in fp32, times both tensor scales, rounded
    once (src/dew/nn/kernels/gemm.py:937-947). The sum is formed exactly and rounded to fp32."""
    left = np.asarray(lhs, np.float64) * np.repeat(np.asarray(lhs_scales, np.float64), 16, axis=-1)
    right = np.asarray(matrices, np.float64) * np.repeat(np.asarray(matrix_scales, np.float64), 16, axis=-1)
    total = np.zeros((left.shape[0], right.shape[1]), F32)
    start = 0
    for group, size in enumerate(np.asarray(group_sizes).tolist()):
        if size:
            total[start:start + size] = (left[start:start + size] @ right[group].T).astype(F32)
        start += size
    total = twice_scaled(total, F32(lhs_scale), F32(matrix_scale))
    if bias is not None:  # each group's bias meets its rows' fp32 sums before the one rounding (projections.py:137-139)
        start = 0
        for group, size in enumerate(np.asarray(group_sizes).tolist()):
            total[start:start + size] = (total[start:start + size] + np.asarray(bias, F32)[group]).astype(F32)
            start += size
    return bf16_round(total) if dtype == "bfloat16" else total


def nvfp4_projection(x, w, group_sizes, *, dtype="bfloat16", bias=None):
    """`x [rows, depth]` and `w [groups, depth, width]` both quantized along the depth (the matrices under one tensor
    scale together), their `nvfp4_block_product` (src/dew/nn/kernels/projections.py:261-275)."""
    rows = nvfp4_quantized(x)
    matrices = nvfp4_quantized(np.swapaxes(np.asarray(w, F32), 1, 2))
    return nvfp4_block_product(*rows, *matrices, group_sizes, dtype=dtype, bias=bias)


E2M3_GRID = np.array([k / 8 for k in range(8)] + [1 + k / 8 for k in range(8)] + [2 + k / 4 for k in range(8)] + [4 + k / 2 for k in range(8)], F32)
"""The magnitudes of FP6 e2m3 (OCP MX: two exponent bits, bias 1, three mantissa bits), by code."""


def e2m3_rounded(values):
    """fp32 values to the nearest e2m3 value, ties to the even code, saturating at +-7.5."""
    values = np.asarray(values, F32)
    magnitude = np.minimum(np.abs(values), F32(7.5))
    above = np.clip(np.searchsorted(E2M3_GRID, magnitude), 1, len(E2M3_GRID) - 1)   # the first grid point at or above
    low, high = E2M3_GRID[above - 1], E2M3_GRID[above]
    up = (high - magnitude < magnitude - low) | ((high - magnitude == magnitude - low) & (above % 2 == 0))
    return (np.sign(values) * np.where(up, high, low)).astype(F32)


def split_rows_fp6(x):
    """bf16 rows as the values `dew_moe_split_rows_fp6` holds them at (no counterpart in the reference, whose products
    take the bf16 rows themselves): `s hi + t lo`, s = the power of two that brings the row's largest magnitude into
    [128, 256) (exponent field clamped to 16 .. 254), hi = e4m3(x / s), t / s = the least power of two that brings the
    largest remainder of each 32 depths within 7.5, lo = e2m3((x / s - hi) / (t / s)). Returns (values fp32 [rows, K],
    scale bytes [rows]). Pinned by its invariants (tests/test_projections.py): exact for every element within two
    binades of its block's largest, within 2^-10 of that largest otherwise, exact on rows of one binade."""
    x = np.asarray(x, F32)
    rows, depth = x.shape
    field = np.clip((np.abs(x).max(axis=1).view(np.uint32) >> 23) & 0xFF, 16, 254).astype(np.int32)
    hi_byte = field - 7
    s = np.ldexp(F32(1), hi_byte - 127)[:, None]
    v = (x / s).astype(F32)
    hi = e4m3_rounded(v)
    rest = (v - hi).astype(F32).reshape(rows, depth // 32, 32)
    most = np.abs(rest).max(axis=-1, keepdims=True)
    bits = most.view(np.uint32)
    power = (bits >> 23).astype(np.int32) - 127 - 2 + ((bits & 0x7FFFFF) > 0x700000)
    power = np.maximum(power, np.maximum(-126, 1 - hi_byte)[:, None, None])
    t_over_s = np.ldexp(F32(1), power)
    lo = e2m3_rounded((rest / t_over_s).astype(F32)) * t_over_s
    values = ((hi.reshape(rest.shape) + lo).reshape(rows, depth) * s).astype(F32)
    return values, hi_byte.astype(np.uint8)


def split_rows_fp6_decoded(split, scale):
    """The values a device buffer of `dew_moe_split_rows_fp6` stands for: `split` uint8 [rows, 2 K] (each 64 depths 128
    bytes: for lane group g, 32 bytes of e4m3 codes of depths 16 g .. 16 g + 15 and 32 + 16 g .. 47 + 16 g, 24 bytes of
    e2m3 codes of depths 32 g .. 32 g + 31 packed six bits each, the second term's e8m0 scale byte), `scale` uint8 [rows]."""
    split = np.asarray(split, np.uint8)
    rows, pitch = split.shape
    steps = split.reshape(rows, pitch // 128, 2, 64)
    table = _e4m3_table()
    hi = table[steps[..., :32]]                                                   # [rows, steps, group, 32]
    first = np.zeros((rows, pitch // 128, 64), F32)
    for g in range(2):
        first[..., 16 * g:16 * g + 16] = hi[:, :, g, :16]
        first[..., 32 + 16 * g:48 + 16 * g] = hi[:, :, g, 16:]
    packed = steps[..., 32:56].astype(np.uint64)                                  # 24 bytes = 32 six-bit codes
    bits = np.zeros((rows, pitch // 128, 2), object)
    codes = np.zeros((rows, pitch // 128, 2, 32), np.int64)
    for i in range(32):
        bit = 6 * i
        lo_byte, shift = bit // 8, bit % 8
        two = packed[..., lo_byte] | (packed[..., min(lo_byte + 1, 23)] << np.uint64(8))
        codes[..., i] = ((two >> np.uint64(shift)) & np.uint64(63)).astype(np.int64)
    magnitudes = E2M3_GRID[codes & 31] * np.where(codes & 32, F32(-1), F32(1))
    t = np.ldexp(F32(1), steps[..., 56].astype(np.int32) - 127)[..., None]
    second = (magnitudes * t).reshape(rows, pitch // 128, 64)
    s = np.ldexp(F32(1), np.asarray(scale, np.uint8).astype(np.int32) - 127)[:, None]
    return ((first * s[:, :, None]) + second).reshape(rows, pitch // 2).astype(F32)


def _e2m3_block_scale(most):
    """The least power of two t with most / t <= 7.5 (e2m3's largest magnitude), kept a normal power of two with an e8m0
    byte of 1 .. 254 (a block of zeros takes the least one)."""
    bits = np.asarray(most, F32).view(np.uint32)
    power = (bits >> 23).astype(np.int32) - 127 - 2 + ((bits & 0x7FFFFF) > 0x700000)
    return np.clip(power, -126, 127)


def split_rows_e2m3_pair(x):
    """bf16 rows as the values `dew_moe_split_rows_e2m3_pair` holds them at (no counterpart in the reference): for every 32
    depths `s hi + t lo`, s = the least power of two with the block's largest magnitude within 7.5 s, hi = e2m3(x / s),
    t the same for the remainders x - s hi, lo = e2m3((x - s hi) / t). Returns (values fp32 [rows, K], the two scales' e8m0
    bytes [rows, K / 32, 2]). Pinned by its invariants (tests/test_projections.py): exact for every element within two
    binades of its block's largest magnitude, within 2^-10 of that magnitude otherwise, exact on blocks of three binades."""
    x = np.asarray(x, F32)
    rows, depth = x.shape
    rest = x.reshape(rows, depth // 32, 32).copy()
    total = np.zeros_like(rest)
    scales = []
    for _ in range(2):
        power = _e2m3_block_scale(np.abs(rest).max(axis=-1, keepdims=True))
        scale = np.ldexp(F32(1), power)
        held = (e2m3_rounded((rest / scale).astype(F32)) * scale).astype(F32)
        total = (total + held).astype(F32)
        rest = (rest - held).astype(F32)
        scales.append((power[..., 0] + 127).astype(np.uint8))
    return total.reshape(rows, depth), np.stack(scales, axis=-1)


def _six_bit_codes(packed):
    """`[..., 24]` bytes as the 32 six-bit codes they pack, in order (code i at bits 6 i .. 6 i + 5, little-endian)."""
    packed = np.asarray(packed, np.uint8).astype(np.uint64)
    codes = np.zeros((*packed.shape[:-1], 32), np.int64)
    for i in range(32):
        low, shift = (6 * i) // 8, (6 * i) % 8
        two = packed[..., low] | (packed[..., min(low + 1, 23)] << np.uint64(8))
        codes[..., i] = ((two >> np.uint64(shift)) & np.uint64(63)).astype(np.int64)
    return codes


def split_rows_e2m3_pair_decoded(split):
    """The values a device buffer of `dew_moe_split_rows_e2m3_pair` stands for, and its scale bytes: `split` uint8
    [rows, 2 K], each 64 depths 128 bytes: for lane group g (depths 32 g .. 32 g + 31) and term t, 24 bytes of e2m3 codes,
    the term's e8m0 byte, 7 unused bytes. Returns (values fp32 [rows, K], scale bytes [rows, K / 32, 2])."""
    split = np.asarray(split, np.uint8)
    rows, pitch = split.shape
    pieces = split.reshape(rows, pitch // 128, 2, 2, 32)               # [rows, steps, group, term, 32 bytes]
    codes = _six_bit_codes(pieces[..., :24])
    magnitudes = E2M3_GRID[codes & 31] * np.where(codes & 32, F32(-1), F32(1))
    scales = pieces[..., 24]
    values = (magnitudes * np.ldexp(F32(1), scales.astype(np.int32) - 127)[..., None]).astype(F32)
    total = (values[:, :, :, 0] + values[:, :, :, 1]).astype(F32)       # [rows, steps, group, 32]
    return total.reshape(rows, pitch // 2), scales.reshape(rows, pitch // 64, 2)


def swiglu(gate, up, *, dtype="bfloat16", limit=None, exp=np.exp):
    """`gated_product('swiglu')` after `swiglu_clamped` (src/dew/nn/activations.py:267-278,327-356):
    bf16 rounds the activation `g * logistic(g)` and then the product with `u`; fp32 rounds nowhere.
    The reference's exp here is the backend's own accurate one, so NumPy's stands for it."""
    gate, up = np.asarray(gate, F32), np.asarray(up, F32)
    if limit is not None:
        gate, up = np.minimum(gate, F32(limit)), np.clip(up, F32(-limit), F32(limit))
    sig = (F32(1) / (F32(1) + exp(-gate).astype(F32)).astype(F32)).astype(F32)
    if dtype != "bfloat16":
        return ((gate * sig).astype(F32) * up).astype(F32)
    gate, up = bf16_round(gate), bf16_round(up)
    sig = (F32(1) / (F32(1) + exp(-gate).astype(F32)).astype(F32)).astype(F32)
    activated = bf16_round((gate * sig).astype(F32))
    return bf16_round((activated * up).astype(F32))


def geglu(gate, up, *, dtype="bfloat16", limit=None, exp=np.exp):
    """`gated_product('geglu')` (src/dew/nn/activations.py:255-278 over `gelu_tanh`, :57-69): the tanh GELU in its logistic
    form `g * logistic(sqrt(8 / pi) (g + 0.044715 g^3))`, every step an fp32 operation in that order, rounded to bf16,
    then the product with `u` rounded again; fp32 rounds nowhere. The clamp as in `swiglu`."""
    gate, up = np.asarray(gate, F32), np.asarray(up, F32)
    if limit is not None:
        gate, up = np.minimum(gate, F32(limit)), np.clip(up, F32(-limit), F32(limit))

    def activated(g):
        cube = ((g * g).astype(F32) * g).astype(F32)
        inner = (F32(np.sqrt(8 / np.pi)) * (g + (F32(0.044715) * cube).astype(F32)).astype(F32)).astype(F32)
        with np.errstate(over="ignore"):
            sig = (F32(1) / (F32(1) + exp(-inner).astype(F32)).astype(F32)).astype(F32)
        return (g * sig).astype(F32)

    if dtype != "bfloat16":
        return (activated(gate) * up).astype(F32)
    gate, up = bf16_round(gate), bf16_round(up)
    return bf16_round((bf16_round(activated(gate)) * up).astype(F32))


GATED_PRODUCTS = {"swiglu": swiglu, "geglu": geglu}


def silu(x, *, dtype="bfloat16", exp=np.exp):
    """`silu` (src/dew/nn/activations.py:100-106): `x * logistic(x)` in fp32, rounded once to the array's dtype. The
    first of `swiglu`'s two roundings; the same stand-in for the backend's exp."""
    x = np.asarray(x, F32)
    if dtype == "bfloat16":
        x = bf16_round(x)
    sig = (F32(1) / (F32(1) + exp(-x).astype(F32)).astype(F32)).astype(F32)
    activated = (x * sig).astype(F32)
    return bf16_round(activated) if dtype == "bfloat16" else activated


def routed_values(x, weights, indices, kernel, *, dtype="bfloat16", factor=None):
    """`RoutedValues.__call__` from the routing on (src/dew/nn/value_experts.py:79-98): each token's chosen projections
    `x @ kernel[e]` (one rounding), each through `silu`, summed under the router's weights in fp32 and rounded once.
    `kernel [E, in, features]` dequantized values. Returns (out [T, features], the slots [T, k, features])."""
    x = np.asarray(x, F32).reshape(-1, np.asarray(x).shape[-1])
    indices = np.asarray(indices).reshape(x.shape[0], -1)
    plan = sorted_by_expert(indices, kernel.shape[0])
    projected = grouped_matmul(x[plan["rows"]], kernel, plan["sizes"], dtype=dtype, factor=factor)
    activated = silu(projected, dtype=dtype)
    slots = np.zeros_like(activated)
    slots[plan["order"]] = activated
    slots = slots.reshape(indices.shape[0], indices.shape[1], -1)
    return combine(slots, np.asarray(weights).reshape(indices.shape), dtype=dtype), slots


def combine(slots, weights, *, dtype="bfloat16"):
    """`ExpertMLP._combine` (src/dew/nn/moe.py:1328-1333): `out[t] = round(sum_j f32(y[t, j]) * w[t, j])`,
    fp32 weights, fp32 sum in slot order, one rounding."""
    slots = np.asarray(slots, F32)
    weights = np.asarray(weights, F32)
    total = np.zeros((slots.shape[0], slots.shape[2]), F32)
    for j in range(slots.shape[1]):
        total = (total + (slots[:, j, :] * weights[:, j, None]).astype(F32)).astype(F32)
    return bf16_round(total) if dtype == "bfloat16" else total


def capacity_admitted(indices, num_experts, capacity_factor):
    """`capacity_positions` and the drop it decides (src/dew/nn/moe.py:832-855, 914-919): `indices [..., length, top_k]`,
    each leading row one sequence; a slot's place is its rank, in slot order, among its sequence's slots of the same
    expert; a queue keeps `int(max(ceil(length * top_k / E) * capacity_factor, capacity_factor))` places, and a slot
    past them takes the sentinel id E. Written as the plain double loop (the definition), not as the reference's
    argsort arithmetic. Returns (admitted ids, capacity)."""
    import math

    indices = np.asarray(indices)
    *_, length, top_k = indices.shape
    capacity = int(max(math.ceil(length * top_k / num_experts) * capacity_factor, capacity_factor))
    flat = indices.reshape(-1, length * top_k)
    admitted = flat.copy()
    for sequence in range(flat.shape[0]):
        queued = np.zeros(num_experts + 1, np.int64)
        for slot in range(flat.shape[1]):
            expert = flat[sequence, slot]
            expert = num_experts if expert < 0 or expert >= num_experts else expert
            if expert == num_experts or queued[expert] >= capacity:
                admitted[sequence, slot] = num_experts
            queued[expert] += 1
    return admitted.reshape(indices.shape).astype(np.int32), capacity


def relu2(x, *, dtype="bfloat16"):
    """`relu2` (src/dew/nn/activations.py:109-111): the square of the ReLU, computed in the compute dtype: one rounding."""
    x = np.asarray(x, F32)
    squared = (np.maximum(x, F32(0)) ** 2).astype(F32)
    return bf16_round(squared) if dtype == "bfloat16" else squared


def expert_mlp(x, weights, indices, gate_w, up_w, down_w, *, dtype="bfloat16", factors=(None, None, None),
               limit=None, capacity_factor=None, activation="swiglu", scale_inputs=False):
    """`ExpertMLP.__call__` (src/dew/nn/moe.py:1335-1353) on one device: sort, gather, paired gate/up
    products, SwiGLU, down product scattered to slot order, combine. The matrices are the dequantized
    `[E, depth, width]` values; `indices [T, k]`, or `[..., length, k]` with `capacity_factor` (each leading row a
    sequence whose experts' queues drop their slots past the capacity: a dropped slot's row is zero). Returns
    (out [T, D], trace dict of the intermediates)."""
    x = np.asarray(x, F32)
    experts = up_w.shape[0]
    if capacity_factor is not None:
        indices, _ = capacity_admitted(indices, experts, capacity_factor)
    indices = np.asarray(indices).reshape(-1, np.asarray(indices).shape[-1])
    x = x.reshape(-1, x.shape[-1])
    weights = np.asarray(weights).reshape(indices.shape)
    plan = sorted_by_expert(indices, experts)
    rows = x[plan["rows"]]   # (rows past the groups, the dropped slots', are multiplied by no matrix: `grouped_matmul` leaves them zero)
    if scale_inputs:
        # Llama 4's placement of the routing weight (src/dew/nn/moe.py:1124-1126, `Llama4TextMoe.forward`): each slot's
        # row times its weight, both in the compute dtype, one rounding; the outputs are then summed unweighted (:1328-1330)
        scale = weights.reshape(-1)[plan["order"]][:, None]
        rows = bf16_round(bf16_round(rows) * bf16_round(scale)) if dtype == "bfloat16" else (rows * scale.astype(F32)).astype(F32)
    up = grouped_matmul(rows, up_w, plan["sizes"], dtype=dtype, factor=factors[1])
    if activation == "relu2":   # Nemotron-H's ungated experts: up_proj, squared ReLU, down_proj (src/dew/nn/moe.py:1319-1322); `gate_w` is None
        gate, hidden = None, relu2(up, dtype=dtype)
    else:
        gate = grouped_matmul(rows, gate_w, plan["sizes"], dtype=dtype, factor=factors[0])
        hidden = GATED_PRODUCTS[activation](gate, up, dtype=dtype, limit=limit)
    projected = grouped_matmul(hidden, down_w, plan["sizes"], dtype=dtype, factor=factors[2])
    slots = np.zeros_like(projected)
    slots[plan["order"]] = projected
    tokens, k = np.asarray(indices).shape
    slots = slots.reshape(tokens, k, -1)
    out = combine(slots, np.ones_like(weights) if scale_inputs else weights, dtype=dtype)
    return out, {**plan, "gate": gate, "up": up, "hidden": hidden, "slots": slots}


def gpt_oss_gating(projected, *, limit=7.0, dtype="bfloat16", exp=np.exp):
    """GPT-OSS's activation of one interleaved projection `[..., 2F]` (src/dew/nn/gpt_oss.py:120-121):
    gate = even columns clamped from above, up = odd columns clamped both ways
    (src/dew/nn/activations.py:327-333), `(up + 1) * quick_gelu(gate)` with `quick_gelu(x) = x * logistic(1.702 x)`
    (src/dew/nn/activations.py:72-74). In bf16 every operation rounds, the Python scalar 1.702 entering as a bf16."""
    projected = np.asarray(projected, F32)
    gate = np.minimum(projected[..., 0::2], F32(limit))
    up = np.clip(projected[..., 1::2], F32(-limit), F32(limit))
    rounded = bf16_round if dtype == "bfloat16" else (lambda v: np.asarray(v, F32))
    slope = rounded(np.asarray(1.702, F32))
    scaled = rounded(gate * slope)
    sig = rounded((F32(1) / (F32(1) + exp(-scaled).astype(F32)).astype(F32)).astype(F32))
    gelu = rounded(gate * sig)
    return rounded(rounded(up + F32(1)) * gelu)


def _biased_matmul(x, w, sizes, bias, *, dtype, factor=None):
    """`grouped_matmul` with each expert's bias added to its rows' fp32 sums before the one rounding
    (src/dew/nn/moe.py:729-742: the bias rounded to the compute dtype, held in fp32)."""
    x = np.asarray(x, F32)
    w = np.asarray(w, F32)
    if dtype == "bfloat16":
        x = bf16_round(x)
    out = np.zeros((x.shape[0], w.shape[2]), F32)
    start = 0
    for group, size in enumerate(np.asarray(sizes).tolist()):
        if size:
            matrix = bf16_round(w[group]) if dtype == "bfloat16" else w[group]
            summed = x[start:start + size] @ matrix
            if factor is not None:
                summed = summed.astype(F32) * F32(factor[group])
            held = np.asarray(bias[group], F32)
            summed = (summed.astype(F32) + (bf16_round(held) if dtype == "bfloat16" else held)).astype(F32)
            out[start:start + size] = summed
        start += size
    return bf16_round(out) if dtype == "bfloat16" else out


def gpt_oss_experts(x, weights, indices, gate_up, gate_up_bias, down, down_bias, *, dtype="bfloat16", limit=7.0,
                    factors=(None, None)):
    """`GptOssExperts.__call__` (src/dew/nn/gpt_oss.py:70-126) on one device: sort the slots by expert, the
    fused biased projection, the clamped gating, the biased down projection back in slot order, and the
    weighted sum over each token's slots. `gate_up [E, D, 2F]` and `down [E, F, D]` are the dequantized values."""
    x = np.asarray(x, F32)
    experts = gate_up.shape[0]
    plan = sorted_by_expert(indices, experts)
    rows = x[plan["rows"]]
    projected = _biased_matmul(rows, gate_up, plan["sizes"], gate_up_bias, dtype=dtype, factor=factors[0])
    hidden = gpt_oss_gating(projected, limit=limit, dtype=dtype)
    output = _biased_matmul(hidden, down, plan["sizes"], down_bias, dtype=dtype, factor=factors[1])
    slots = np.zeros_like(output)
    slots[plan["order"]] = output
    tokens, k = np.asarray(indices).shape
    slots = slots.reshape(tokens, k, -1)
    return combine(slots, weights, dtype=dtype), {**plan, "projected": projected, "hidden": hidden, "slots": slots}


def gpt_oss_mlp(x, router_kernel, router_bias, gate_up, gate_up_bias, down, down_bias, *, top_k_count,
                dtype="bfloat16", limit=7.0, factors=(None, None)):
    """`GptOssMLP.__call__` (src/dew/nn/gpt_oss.py:155-171): logits = x @ kernel + bias in fp32, the k largest
    logits, the softmax of the chosen logits (`renormalized_softmax`, src/dew/nn/moe.py:194-199), the experts."""
    x = np.asarray(x, F32)
    flat = x.reshape(-1, x.shape[-1])
    logits = (router_logits(bf16_round(flat) if dtype == "bfloat16" else flat, router_kernel)
              + np.asarray(router_bias, F32)).astype(F32)
    weights, indices = route(logits, top_k_count, score_function="softmax", normalize_weights=True)
    out, trace = gpt_oss_experts(flat, weights, indices, gate_up, gate_up_bias, down, down_bias, dtype=dtype,
                                 limit=limit, factors=factors)
    trace.update(logits=logits, weights=weights, indices=indices)
    return out.reshape(*x.shape[:-1], -1), trace


def gated_mlp(x, gate_w, up_w, down_w, *, dtype="bfloat16"):
    """The dense shared expert (`GatedMLP`, src/dew/nn/mlp.py:106,239): SwiGLU MLP on every token, the same
    rounding points as one expert holding all rows."""
    sizes = [np.asarray(x).shape[0]]
    gate = grouped_matmul(x, np.asarray(gate_w)[None], sizes, dtype=dtype)
    up = grouped_matmul(x, np.asarray(up_w)[None], sizes, dtype=dtype)
    return grouped_matmul(swiglu(gate, up, dtype=dtype), np.asarray(down_w)[None], sizes, dtype=dtype)


def gated_rows(x, kernel, rows):
    """`shared * logistic(shared_expert_gate(x))` (src/dew/nn/moe.py:1469-1475, 1499-1502) under a bf16 compute dtype: the
    gate's `Dense(1)` promotes its fp32 kernel to bf16 (flax's `promote_dtype` under `dtype`), multiplies bf16 operands
    with an fp32 sum and returns bf16; the logistic is formed in fp32 and rounded once to bf16
    (src/dew/nn/activations.py:85-98); the bf16 product with the shared expert's output is rounded once."""
    x = np.asarray(x, F32)
    kernel = bf16_round(np.asarray(kernel, F32).reshape(-1))
    logit = bf16_round((x.astype(np.float64) @ kernel.astype(np.float64)).astype(F32))
    gate = bf16_round(logistic(logit))   # (fp32, the fixed-sequence exponential: the device kernel's own steps, so the gates agree bit for bit)
    return bf16_round((np.asarray(rows, F32) * gate[:, None]).astype(F32))


def gated_rows_added_f32(x, kernel, shared, routed):
    """`routed + shared * logistic(shared_expert_gate(x))` (src/dew/nn/moe.py:1469-1475, 1497-1503) where the layer states no
    compute dtype: the gate's `Dense(1)` promotes the bf16 token to its fp32 kernel (flax's `promote_dtype` without a
    `dtype`), so the logit, its logistic, the product with the shared expert's bf16 rows and the sum with the routed
    experts' bf16 rows are float32, each operation rounded once. (The logit's sum in float64, rounded once: the device
    kernel's own steps. Like the bf16 gate's, these rounding points are read from the sources and pinned by no fixture.)"""
    x = np.asarray(x, F32)
    kernel = np.asarray(kernel, F32).reshape(-1)
    logit = (x.astype(np.float64) @ kernel.astype(np.float64)).astype(F32)
    gated = (np.asarray(shared, F32) * logistic(logit)[:, None]).astype(F32)
    return (np.asarray(routed, F32) + gated).astype(F32)


def sparse_mlp(x, logits, gate_w, up_w, down_w, *, top_k_count, dtype="bfloat16", shared=None,
               factors=(None, None, None), limit=None, scale_inputs=False, shared_gate=None, **router):
    """`SparseMLP.__call__` (src/dew/nn/moe.py:1488-1503) from the router logits on: route, routed
    experts, plus the shared expert's output (`shared` = its three dense matrices)."""
    weights, indices = route(logits, top_k_count, **router)
    routed, trace = expert_mlp(x, weights, indices, gate_w, up_w, down_w, dtype=dtype, factors=factors,
                               limit=limit, scale_inputs=scale_inputs)
    trace.update(weights=weights, indices=indices)
    if shared is not None:
        apart = gated_mlp(x, *shared, dtype=dtype)
        if shared_gate is not None:      # Qwen2-MoE's scalar gate on the shared expert (bf16 compute dtype)
            apart = gated_rows(x, shared_gate, apart)
        both = routed + apart
        routed = bf16_round(both) if dtype == "bfloat16" else both.astype(F32)
    return routed, trace


def relative_errors(got, want, floor=None):
    """The two error figures reported per config: the reference's own `max|d| / max|want|`
    (tools/benchmark_kernels.py:143-144) and the element-wise max relative error `|d| / max(|want|, floor)`,
    the floor by default rms(want): an output far below the rms is a cancellation of its k weighted expert
    rows, each already rounded to bf16, so its own magnitude says nothing of the error it can carry."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    scale = np.abs(want).max()
    floor = np.sqrt(np.mean(want ** 2)) if floor is None else floor
    delta = np.abs(got - want)
    return float(delta.max() / scale), float((delta / np.maximum(np.abs(want), floor)).max())
