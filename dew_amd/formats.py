"""The quantized expert banks the MoE layer holds, in the reference's own storage layouts, so a checkpoint
packed for it is read here unchanged.

`NvFp4` mirrors the reference's bank (src/dew/nn/kernels/formats.py:27-137): K-major uint32 `words
[E, N, K/8]`, each the GF(2)-encoded word (src/dew/algebra/bits.py:696-705) of eight E2M1 codes taken in
the staged depth order (word w of a 128-deep group holds depths 128g + 16j + w, j = 0..7;
src/dew/nn/kernels/templates/gemm/packed.py:27-33); `scales [E, N, K/16]` float8_e4m3fn bytes in natural
depth order; `scale [E]` fp32; `form` the 8-byte digest of the encoder that packed the words. MXFP4
checkpoints enter through `NvFp4.of(*codecs.mxfp4_as_nvfp4(...))`, as the reference loads them
(src/dew/interop/quantized_loads.py:106-143).

`Fp8Blocks` / `Fp8Channels` hold e4m3 codes `[E, K, N]` with 128x128-block or per-output-channel fp32
scales (a DeepSeek-style checkpoint's `weight` / `weight_scale_inv`, src/dew/interop/codecs.py:670-703).

The HIP kernels read a one-time device re-layout of these banks (`prepared.py`); the encoder is an
invertible GF(2) map, so that re-layout is exact.
"""

import dataclasses
import hashlib

import torch

NVFP4_ENCODER = (
    0x4000100, 0x8000202, 0x4040401, 0x2800080, 0x1000000, 0x2000000, 0x4000000, 0x8000002,
    0x4040001, 0x20000808, 0x4010000, 0x8020002, 0x4000001, 0x8000000, 0x4040005, 0x20000008,
    0x40001000, 0x80002020, 0x40404010, 0x20080008, 0x10000000, 0x20000000, 0x40000000, 0x80000020,
    0x40400010, 0x2008080, 0x40100000, 0x80200020, 0x40000010, 0x80000000, 0x40400050, 0x2000080)
"""Stored bit i = parity(natural word & NVFP4_ENCODER[i]) (src/dew/algebra/bits.py:702-705)."""

FORM_HEX = hashlib.sha256(",".join(map(str, NVFP4_ENCODER)).encode()).hexdigest()[:16]
"""Version of the stored word layout (src/dew/algebra/bits.py:306-311): 7fb7f1b609cea47a."""

NVFP4_OWED = 256.0
NVFP4_GROUP = 128
NVFP4_STAGE = 256
"""An NVFP4 matrix's depth is whole 256s (src/dew/nn/kernels/formats.py:139)."""


def form_bytes(device=None) -> torch.Tensor:
    return torch.tensor(list(bytes.fromhex(FORM_HEX)), dtype=torch.uint8, device=device)


def staged_rows(depth: int, device=None) -> torch.Tensor:
    """The depth each packed row holds: row `8w + j` of group g holds depth `128g + 16j + w`
    (src/dew/nn/kernels/formats.py:144-155)."""
    if depth % NVFP4_GROUP:
        raise ValueError(f"an NVFP4 matrix's depth is whole {NVFP4_GROUP}-deep groups, not {depth}")
    index = torch.arange(depth, device=device)
    group, within = index // NVFP4_GROUP, index % NVFP4_GROUP
    return NVFP4_GROUP * group + 16 * (within % 8) + within // 8


def _encoder_tables(device):
    """The encoder as four 256-entry tables, one a byte of the natural word: it is GF(2)-linear, so a
    word's image is the xor of its bytes' images."""
    tables = []
    for byte in range(4):
        column = []
        for value in range(256):
            natural = value << (8 * byte)
            column.append(sum((bin(natural & mask).count("1") & 1) << bit for bit, mask in enumerate(NVFP4_ENCODER)))
        tables.append(torch.tensor(column, dtype=torch.int64, device=device))
    return tables


def encoded_words(nibbles: torch.Tensor) -> torch.Tensor:
    """Eight nibbles `[..., 8]` (code j at natural bits 4j..4j+3) as the stored word, int32 bits
    `[...]` (`bits.packed`, src/dew/algebra/bits.py:921-931)."""
    pairs = nibbles.to(torch.int64).reshape(*nibbles.shape[:-1], 4, 2)
    natural_bytes = pairs[..., 0] | (pairs[..., 1] << 4)
    tables = _encoder_tables(nibbles.device)
    stored = tables[0][natural_bytes[..., 0]]
    for byte in range(1, 4):
        stored = stored ^ tables[byte][natural_bytes[..., byte]]
    return torch.where(stored >= 2 ** 31, stored - 2 ** 32, stored).to(torch.int32)


@dataclasses.dataclass(frozen=True)
class NvFp4:
    """A bank of NVFP4 expert matrices standing for `W [E, K, N]`; fields as the module docstring lays them
    out. `words` is held as int32 (torch has no uint32 arithmetic); the bits are the reference's uint32."""

    words: torch.Tensor
    scales: torch.Tensor
    scale: torch.Tensor
    form: torch.Tensor = None

    def __post_init__(self):
        if self.form is None:
            object.__setattr__(self, "form", form_bytes(self.words.device))

    @classmethod
    def of(cls, codes: torch.Tensor, scales: torch.Tensor, scale: torch.Tensor) -> "NvFp4":
        """The bank of `codes [E, K, N]` (uint8 nibbles, sign bit 3, natural depth order), block scales
        `[E, K/16, N]` (e4m3 bytes) and tensor scales `[E]`: packed in the staged order, K-major
        (src/dew/nn/kernels/formats.py:82-96)."""
        if codes.ndim == 2:
            codes, scales, scale = codes[None], scales[None], scale.reshape(1)
        experts, depth, width = codes.shape
        if depth % NVFP4_STAGE:
            raise ValueError(f"an NVFP4 matrix's depth is whole {NVFP4_STAGE}s, not {depth}")
        ordered = codes[:, staged_rows(depth, codes.device), :]                       # [E, K (staged), N]
        words = encoded_words(ordered.transpose(1, 2).reshape(experts, width, depth // 8, 8))
        return cls(words.contiguous(), scales.transpose(1, 2).contiguous().view(torch.uint8),
                   scale.to(torch.float32).reshape(experts).contiguous())

    @classmethod
    def quantized(cls, weight: torch.Tensor) -> "NvFp4":
        """`weight [E, K, N]` quantized to NVFP4, each expert's matrix on its own
        (src/dew/nn/kernels/formats.py:71-80)."""
        from . import codecs

        parts = [codecs.nvfp4_coded(matrix) for matrix in weight]
        return cls.of(*(torch.stack(field) for field in zip(*parts, strict=True)))

    def checked(self) -> "NvFp4":
        """Itself where its words are this form's; refused otherwise (src/dew/nn/kernels/formats.py:49-69)."""
        held = self.form.reshape(-1, 8).cpu()
        found = {bytes(row.tolist()).hex() for row in held}
        if found != {FORM_HEX}:
            raise ValueError(f"NVFP4 words packed by form version {', '.join(sorted(found))}, where this "
                             f"library decodes form version {FORM_HEX}: repack them from the source weights")
        return self

    @property
    def shape(self):
        experts, width, words = self.words.shape
        return (experts, 8 * words, width)

    @property
    def dtype(self):
        """The dtype its decode yields and it is multiplied as (src/dew/nn/kernels/formats.py:115-118)."""
        return torch.bfloat16

    @property
    def factor(self) -> torch.Tensor:
        """2^8 times each expert's tensor scale, owed to the accumulator
        (src/dew/nn/kernels/formats.py:132-137)."""
        return self.scale.to(torch.float32) * NVFP4_OWED

    def to(self, device) -> "NvFp4":
        return NvFp4(self.words.to(device), self.scales.to(device), self.scale.to(device), self.form.to(device))


@dataclasses.dataclass(frozen=True)
class Fp8Blocks:
    """FP8 e4m3 codes `[E, K, N]` (uint8) with fp32 `scale_inv [E, ceil(K/128), ceil(N/128)]`: value
    `f32(code) * scale_inv[k // 128, n // 128]`, rounded to the compute dtype before the product, as the
    reference dequantizes such a checkpoint at load (src/dew/interop/codecs.py:638-648,670-703)."""

    codes: torch.Tensor
    scale_inv: torch.Tensor
    kmajor: bool = False
    """The tensors as such a checkpoint stores them, stacked by expert: `codes [E, N, K]` (each expert's `weight [out,
    in]`) and `scale_inv [E, N/128, K/128]`; the bank still stands for `W [E, K, N]`, and its re-layout for the matrix
    cores reads them where they lie."""

    @classmethod
    def quantized(cls, weight: torch.Tensor) -> "Fp8Blocks":
        from . import codecs

        return cls(*codecs.fp8_block_cast(weight, (128, 128)))

    @property
    def shape(self):
        experts, first, second = self.codes.shape
        return (experts, second, first) if self.kmajor else (experts, first, second)

    @property
    def dtype(self):
        return torch.bfloat16

    def to(self, device) -> "Fp8Blocks":
        return Fp8Blocks(self.codes.to(device), self.scale_inv.to(device), self.kmajor)


@dataclasses.dataclass(frozen=True)
class Mxfp4Blocks:
    """An MXFP4 checkpoint's expert bank as the checkpoint stores it (gpt-oss's `*_blocks` / `*_scales`,
    src/dew/interop/codecs.py:193-224): `blocks [E, N, K/32, 16]` uint8, two E2M1 codes a byte (low nibble the even
    element), and `scales [E, N, K/32]` E8M0 bytes; standing for `W [E, K, N]`. The reference turns such a bank into
    its `NvFp4` on the host (`mxfp4_as_nvfp4`, src/dew/interop/codecs.py:265-284); here the device re-layout takes
    these bytes straight to the same prepared bank (`DEW_MOE_W_MXFP4_BLOCKS`)."""

    blocks: torch.Tensor
    scales: torch.Tensor

    def __post_init__(self):
        if self.blocks.ndim != 4 or self.blocks.shape[-1] != 16 or tuple(self.scales.shape) != tuple(self.blocks.shape[:3]):
            raise ValueError(f"an MXFP4 bank is blocks [E, N, K/32, 16] with scales [E, N, K/32], got {tuple(self.blocks.shape)} "
                             f"and {tuple(self.scales.shape)}")

    @property
    def shape(self):
        experts, width, groups, _ = self.blocks.shape
        return (experts, 32 * groups, width)

    @property
    def dtype(self):
        return torch.bfloat16

    def to(self, device) -> "Mxfp4Blocks":
        return Mxfp4Blocks(self.blocks.to(device), self.scales.to(device))


@dataclasses.dataclass(frozen=True)
class Fp8Channels:
    """FP8 e4m3 codes `[E, K, N]` (uint8) with one fp32 scale per output channel `[E, N]`."""

    codes: torch.Tensor
    scales: torch.Tensor

    @classmethod
    def quantized(cls, weight: torch.Tensor) -> "Fp8Channels":
        from . import codecs

        return cls(*codecs.fp8_channel_cast(weight))

    @property
    def shape(self):
        return tuple(self.codes.shape)

    @property
    def dtype(self):
        return torch.bfloat16

    def to(self, device) -> "Fp8Channels":
        return Fp8Channels(self.codes.to(device), self.scales.to(device))


@dataclasses.dataclass(frozen=True)
class Bf16:
    """Unquantized matrices `[E, K, N]` bf16 as the reference's experts hold them (`experts/*_proj/kernel`,
    src/dew/nn/moe.py:1231-1235): the grouped product's plain operand (`expert_projection`,
    src/dew/nn/moe.py:666-726), wrapped so that its one-time re-layout for the matrix cores is kept with it."""

    weights: torch.Tensor
    transposed: bool = False   # the same memory as the matrices of the transposed product (an input gradient's)

    def __post_init__(self):
        if self.weights.dtype != torch.bfloat16 or self.weights.ndim != 3:
            raise ValueError(f"a bf16 bank is bfloat16 [E, K, N], not {self.weights.dtype} {tuple(self.weights.shape)}")

    @property
    def shape(self):
        experts, depth, width = self.weights.shape
        return (experts, width, depth) if self.transposed else (experts, depth, width)

    @property
    def dtype(self):
        return torch.bfloat16

    @property
    def T(self) -> "Bf16":
        """The bank of every matrix's transpose, over the same memory: what an input gradient multiplies by."""
        return Bf16(self.weights, not self.transposed)

    def to(self, device) -> "Bf16":
        return Bf16(self.weights.to(device), self.transposed)


@dataclasses.dataclass(frozen=True)
class MxFp8:
    """An MXFP8 bank of matrices, K-major as a product reads them (the reference's `MxFp8` operand,
    src/dew/nn/kernels/formats.py:186-194): e4m3 `codes [E, N, K]` (uint8) and one E8M0 `scales [E, N, K / 32]` byte
    (uint8) every 32 depths, value = code * 2^(byte - 127). Standing for `W [E, K, N]`."""

    codes: torch.Tensor
    scales: torch.Tensor

    @classmethod
    def quantized(cls, weight: torch.Tensor) -> "MxFp8":
        """`weight [E, K, N]` quantized along the depth by OCP MX's rule (`MxFp8.quantized`,
        src/dew/nn/kernels/formats.py:195-229): each 32 depths' scale 2^(largest magnitude's exponent - 8), codes
        rounded to e4m3, ties to even, saturating at +-448; a block of zeros takes the least scale."""
        matrices = weight.to(torch.float32).transpose(1, 2).contiguous()      # [E, N, K]
        experts, width, depth = matrices.shape
        blocks = matrices.reshape(experts, width, depth // 32, 32)
        largest = blocks.abs().amax(dim=-1, keepdim=True)
        field = (largest.contiguous().view(torch.int32) >> 23) & 0xFF          # 0 for zero and subnormal magnitudes
        byte = (field - 8).clamp(0, 254)
        inverse = ((254 - byte) << 23).view(torch.float32)                     # 2^(127 - byte)
        codes = (blocks * inverse).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
        return cls(codes.reshape(experts, width, depth).contiguous(), byte[..., 0].to(torch.uint8).contiguous())

    @property
    def shape(self):
        experts, width, depth = self.codes.shape
        return (experts, depth, width)

    @property
    def dtype(self):
        return torch.bfloat16

    def to(self, device) -> "MxFp8":
        return MxFp8(self.codes.to(device), self.scales.to(device))


def stacked(banks):
    """Banks of one format and one matrix shape as one bank along the expert axis (the routed experts and, behind
    them, an always-on expert the same launches multiply as one more group), or None where they do not stack."""
    first = banks[0]
    if any(type(bank) is not type(first) or tuple(bank.shape[1:]) != tuple(first.shape[1:]) for bank in banks):
        return None
    if isinstance(first, (Fp8Blocks, Bf16)) and any(getattr(bank, "kmajor", False) != getattr(first, "kmajor", False)
                                                   or getattr(bank, "transposed", False) != getattr(first, "transposed", False) for bank in banks):
        return None
    if not dataclasses.is_dataclass(first) or isinstance(first, Layered):
        return None
    joined = {}
    for field in dataclasses.fields(first):
        value = getattr(first, field.name)
        if field.name == "form":
            continue
        joined[field.name] = torch.cat([getattr(bank, field.name) for bank in banks]) if torch.is_tensor(value) else value
    return type(first)(**joined)


@dataclasses.dataclass(frozen=True)
class Layered:
    """An expert kernel read in place from a run's stack (src/dew/nn/moe.py:595-606): `stack` the bank of every
    layer's experts along one axis (`[layers * E, K, N]`, any of the quantized formats or its prepared form) and
    the `layer` read of `layers`. The grouped launch reads the layer's matrices where they lie."""

    stack: object
    layer: int
    layers: int

    @property
    def shape(self):
        total, depth, width = self.stack.shape
        return (total // self.layers, depth, width)

    @property
    def dtype(self):
        return torch.bfloat16
