// Grouped GEMM over expert-sorted rows on the gfx950 matrix cores: bf16 activations times quantized expert
// weights dequantized to bf16 in registers (exactly the values the reference's load produces), fp32
// accumulation in v_mfma_f32_32x32x16_bf16, one rounding to bf16.
//
//   out[scatter[i], :] = bf16( sum_k x[gather[i], k] * W[e(i)][k, :] + bias[e(i)] )   (expert_projection)
//   hidden[i, :] = swiglu(x[gather[i]] @ Wg[e], x[gather[i]] @ Wu[e])                 (paired gate/up + epilogue)
//   hidden[i, :] = gated pairs of one interleaved bank's columns                       (GPT-OSS's gate_up)
//
// Work decomposition: a 256-thread block (4 wavefronts side by side along the columns) owns a BM-row x BN-column
// tile of one expert's group (two such tiles, gate and up, when paired) and walks the depth in 64-deep steps.
// Tiles are enumerated on the device from `offsets` (no host read of the routing); experts with no rows own no
// tiles. The finished tile is staged in the LDS and leaves as whole rows.
//
// For MXFP4 banks there is a second operand path (kFormatMxSplit): activation rows split beforehand into two e4m3
// terms and multiplied by the stored FP4 codes with v_mfma_scale_f32_32x32x64_f8f6f4, nothing dequantized.
//
// Operand paths, shaped by what the LDS of this chip costs (measured: ds_read_b128 ~230 B/clk a CU,
// ds_write_b128 ~70 B/clk):
//   A (activation rows, gathered by index): global -> LDS directly (global_load_lds_dwordx4, no registers and
//     no ds_write, two steps ahead into a ring of three stages; 128-byte rows, chunk index xor-swizzled so
//     the fragment reads are conflict-free) -> ds_read_b128 fragments.
//   B (weights): never touch the LDS. The prepared bank is in MFMA-fragment order, so each wavefront loads the
//     16-byte pieces of its own 32-column tiles straight from global memory (1 KiB coalesced per load) and
//     dequantizes one 16-deep slice at a time in the shadow of the previous slice's matrix instructions.
//     A lane's 16 bytes hold a run of consecutive depths, so the depth order inside a 64-deep step is permuted
//     (the same permutation on the A side: only the LDS chunk a lane reads changes).
#include <mutex>
#include <type_traits>
#include <utility>

#include "common.h"

namespace dew {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;  // a 16-byte register quad (native vector: stays in VGPRs)
typedef __attribute__((ext_vector_type(8))) int i32x8_t;       // an operand of the scaled matrix instruction
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

// Kernel-side format of an MXFP4 bank multiplied by activation rows already split into two e4m3 terms
// (dew_moe_split_rows): v_mfma_scale_f32_32x32x64_f8f6f4 takes the FP4 codes and their power-of-two block scales
// as they are stored, so the weights are not dequantized at all.
constexpr int kFormatMxSplit = 16;
constexpr int kFormatMxSplitBlocks = 17;  // the same with one activation scale per row and 128 depths, not per row
// Kernel-side format of an FP8 128 x 128 block bank whose scales are powers of two, multiplied by rows quantized to
// e4m3 a 1 x 128 tile at a time under power-of-two scales (dew_moe_quantize_rows_fp8): the blockwise FP8 recipe's
// product. The same instruction takes both operands' codes and scales as stored; a step is 128 depths, its two
// 64-deep halves taking the places of the split rows' two terms.
constexpr int kFormatFp8Rows = 18;
// Kernel-side format of an MXFP8 bank (DEW_MOE_W_MXFP8: e4m3 codes, one E8M0 scale per column and 32 depths)
// multiplied by MXFP8 rows (dew_moe_quantize_rows_mxfp8): OCP MX as the instruction defines it, each lane handing
// in the scale byte of its row (column) and 32-deep block. The rows' scale bytes ride the A ring, a dword a row a
// step; the weights' come with their atoms, a dword a column a step.
constexpr int kFormatMxFp8Rows = 19;
// The same instruction stream as a kernel gradient (each group's rows contracted: out[g] = lhs_t[:, group g's tokens] x
// rhs_t[:, group g's tokens]^T): the "rows" are the lhs_t's (the same `window_rows` of them for every group), the
// "bank" is the rhs_t quantized along the tokens and laid out as an MXFP8 bank of one expert whose depth is all the
// tokens, and group g contracts the window of 128-token blocks its offsets name (dew_moe_kernel_gradient_mxfp8).
constexpr int kFormatMxFp8Window = 20;
// The kernel gradient of bf16 operands (the reference's `gemm_t`): lhs_t rows [depth, tokens] bf16 and the rhs_t as a
// DEW_MOE_W_BF16 bank of one expert whose depth is all the tokens; windows in whole 64-token steps.
constexpr int kFormatBf16Window = 21;
// kFormatMxSplit with the second term in FP6: rows split by dew_moe_split_rows_fp6 into an e4m3 term and an e2m3 term
// under one power-of-two scale every 32 depths (the scaled instruction's own granularity). The FP6 x FP4 instruction
// takes half the cycles of the FP8 x FP4 one, so a product's two instructions take three quarters of the time; the
// second term is exact only for elements within two binades of their 32-deep block's largest (see split.hip).
constexpr int kFormatMxSplit6 = 22;
// kFormatMxSplit with both terms in FP6 (dew_moe_split_rows_e2m3_pair: each term's power-of-two scale every 32 depths lies
// with its codes, no scale a row): two FP6 x FP4 instructions a product, the time of one FP8 x FP4 instruction.
constexpr int kFormatMxSplit66 = 24;
// Kernel-side format of a general NVFP4 bank (e4m3 block scales with mantissas) multiplied by activation rows brought to
// f16 under one power-of-two scale a row (dew_moe_rows_f16), on v_mfma_f32_32x32x16_f16. A code times its block scale has
// at most six significant bits and lies in 2^-10 .. 2688: exact in f16, formed by one packed conversion and one packed f16
// multiply for two codes (the bf16 form needs the multiply in fp32 and a packed rounding: twice the vector instructions).
// Every product is the bf16 path's product times a power of two and the sums are fp32 either way, so the launch returns
// the bf16-operand launch's bits.
constexpr int kFormatNvF16 = 23;

constexpr int BK = 64;
constexpr int kThreads = 256;
constexpr int kChunksPerRow = BK / 8;  // 16-byte chunks in an LDS row
constexpr int kMaxDepthBlocks = 256;   // FP8 128 x 128 blocks: depth up to 32768
constexpr int kMaxBlockScaleDepth = 24576;  // block-scaled split rows: 256 rows x 192 scale bytes fit the LDS behind the ring

struct BankView {
  const uint8_t* codes;
  const void* scales;
  const float* tensor_scale;
};

struct GemmParams {
  const bf16_t* x;
  const int32_t* gather;
  const int32_t* offsets;  // [experts + 1] exclusive prefix of the group sizes, or null where `sizes` is given
  const int32_t* sizes;    // [experts] group sizes as jax.lax.ragged_dot takes them: the prefix is then formed in the tile search
  const int32_t* scatter;
  BankView w0, w1;
  bf16_t* out;
  const uint8_t* a_scale;  // split activations: each source row's e8m0 scale, or its row of block_scale_pitch(depth) of them
  uint8_t* out_scale;      // split output: each written row's block_scale_pitch(width) e8m0 scales, one for 128 columns
  const float* bias;  // [experts, width] fp32, or null
  int round_bias;     // the bias is a parameter of a bf16 product: rounded to bf16 as it is read (a quantized-rows recipe's stays fp32)
  float limit;        // the interleaved gated epilogue's clamp; a paired launch's (0: none)
  int gating;         // a paired launch's gate: DEW_MOE_GATE_SILU (SwiGLU) or DEW_MOE_GATE_GELU_TANH (GeGLU)
  int experts, depth, width, rows, m_tile_bound;
  // A launch normally multiplies every group in tiles of its BM rows, the last of a group partly empty. Where that
  // waste matters two launches share the groups: the taller tiles' launch leaves a last tile that would hold at most
  // skip_tails rows to a launch of tiles that many rows tall, which multiplies (tail_of = the taller tile's rows)
  // only those last rows, the ones past a group's whole tiles of tail_of rows where they are at most its own BM.
  int skip_tails, tail_of;
  // A kernel gradient (kFormatMxFp8Window): every group multiplies the same window_rows rows over its own window of
  // the depth, tokens windows[g] .. windows[g + 1] in whole 128s; `depth` is then all the tokens.
  const int32_t* windows;
  int window_rows;
  float* out_f32;  // the product in fp32 (kPlainF32) instead of `out`
  int group_m;     // m-tiles of a chunk of 8 group_m tiles that one XCD's resident blocks cover together (set by launch_tile)
  const float* factor0;  // a kernel gradient's fp32 sums times *factor0 * *factor1 before the rounding (each may be null):
  const float* factor1;  // the tensor scales of NVFP4 operands
};

// What the epilogue writes: the rounded product (plus bias); SwiGLU of two banks' products; for one bank whose
// columns interleave gate (even) and up (odd), the clamped quick-GELU gating of each column pair; or the SwiGLU of
// two banks' products already split into two e4m3 terms under one scale per row and 128 columns, which is what the
// next product's scaled matrix instructions read (kFormatMxSplitBlocks).
enum Epilogue { kPlain = 0, kSwigluOfTwo = 1, kInterleavedGated = 2, kSwigluOfTwoSplit = 3, kPlainF32 = 4 };

// LDS index of 16-byte chunk `chunk` of row `row` (128-byte rows). The chunk is xor-swizzled by
// f(row) = ((row >> 1) & 7) ^ ((row & 1) << 2), chosen against the measured service order of gfx950's LDS:
// ds_read_b128 serves 16 lanes a pass over 64 banks, the passes being lanes {0-3,12-15,20-23,24-27},
// {4-7,8-11,16-19,28-31} and the same + 32; ds_write_b128 serves 8 consecutive lanes a pass over 128 bytes.
// With lane = row (mod 32) on the read side, f is injective on every read pass's rows of one parity, and a
// store pass writes the 8 chunks of one row, so fragment reads and stores are conflict-free.
__device__ __forceinline__ int swizzled(int row, int chunk) {
  return row * kChunksPerRow + (chunk ^ (((row >> 1) & 7) ^ ((row & 1) << 2)));
}

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  bf16x2_t pair = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
  return __builtin_bit_cast(uint32_t, pair);
}

// Eight e4m3 codes (two dwords) times one fp32 scale -> one bf16x8 fragment: bf16(f32(code) * scale), the
// value the reference's dequantize-then-cast produces (src/dew/interop/codecs.py:670-703; gemm.py:1067-1071).
__device__ __forceinline__ bf16x8_t fragment_fp8(uint32_t w0, uint32_t w1, float scale) {
  const f32x2_t a = __builtin_amdgcn_cvt_pk_f32_fp8(w0, false), b = __builtin_amdgcn_cvt_pk_f32_fp8(w0, true);
  const f32x2_t c = __builtin_amdgcn_cvt_pk_f32_fp8(w1, false), d = __builtin_amdgcn_cvt_pk_f32_fp8(w1, true);
  return __builtin_bit_cast(bf16x8_t, u32x4_t{pack_bf16(a.x * scale, a.y * scale), pack_bf16(b.x * scale, b.y * scale),
                                              pack_bf16(c.x * scale, c.y * scale), pack_bf16(d.x * scale, d.y * scale)});
}

// Eight E2M1 nibbles (one dword) under one e4m3 block scale already over 2^8 -> one bf16x8 fragment; each
// product code * scale / 2^8 is exact in bf16 (src/dew/nn/kernels/formats.py:108-113).
__device__ __forceinline__ bf16x8_t fragment_fp4(uint32_t word, float scale) {
  const f32x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0), b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
  const f32x2_t c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2), d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
  return __builtin_bit_cast(bf16x8_t, u32x4_t{pack_bf16(a.x * scale, a.y * scale), pack_bf16(b.x * scale, b.y * scale),
                                              pack_bf16(c.x * scale, c.y * scale), pack_bf16(d.x * scale, d.y * scale)});
}

// The same for a bank whose block scales are all powers of two (an MXFP4 checkpoint's): the hardware
// conversion applies the scale's exponent itself, one instruction for two codes, exactly.
__device__ __forceinline__ bf16x8_t fragment_fp4_pow2(uint32_t word, float scale) {
  return __builtin_bit_cast(bf16x8_t, u32x4_t{
      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 0)),
      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 1)),
      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 2)),
      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(word, scale, 3))});
}

// The same eight codes as f16 values times the block scale itself (an e4m3 value is exact in f16, and so is its product
// with an E2M1 code): one packed conversion and one packed multiply for two codes.
__device__ __forceinline__ bf16x8_t fragment_fp4_f16(uint32_t word, _Float16 scale) {
  const f16x2_t both = {scale, scale};
  const f16x2_t a = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 0) * both, b = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 1) * both;
  const f16x2_t c = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 2) * both, d = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 3) * both;
  return __builtin_bit_cast(bf16x8_t, u32x4_t{__builtin_bit_cast(uint32_t, a), __builtin_bit_cast(uint32_t, b),
                                              __builtin_bit_cast(uint32_t, c), __builtin_bit_cast(uint32_t, d)});
}

// Bytes of one row's block scales (one e8m0 byte for 128 elements), padded to whole 16-byte loads.
__host__ __device__ constexpr int block_scale_pitch(int elements) { return (elements / 128 + 15) / 16 * 16; }

// Dynamic LDS of a block: the three-stage ring of A rows, or the staged output tile (the 32-row tile of 256 columns) with
// the table of its rows' destinations behind it, where that is larger.
template <int BM, int BN, int MODE>
constexpr size_t shared_bytes() {
  constexpr size_t ring = 3 * static_cast<size_t>(BM) * BK * 2;
  constexpr size_t staged = static_cast<size_t>(BM / ((BN == 256 && BM > 32) ? 2 : 1)) * ((MODE == 2 ? BN / 2 : BN) / 2 + 4) * 4 + BM * 4;
  return ring > staged ? ring : staged;
}

// f(integral_constant<B>), f(integral_constant<B + 1>), ...: a loop whose index is a constant expression in its body.
template <int B, int... Is, class F>
__device__ __forceinline__ void static_range(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, B + Is>{}), ...);
}

// Instruction order of one phase of the main loop, stated to the scheduler: `MFMAS` matrix instructions in a
// row, the phase's `DSR` operand reads issued one behind each of the first of them (so they are long done
// when the next phase multiplies them), and the phase's other work (vector ALU, LDS stores, global loads)
// dealt evenly into the shadows of all of them. Masks: 0x8 MFMA, 0x100 DS read, 0x200 DS write, 0x2 VALU,
// 0x20 VMEM read.
template <int M, int MFMAS, int DSR, int DSW, int VALU, int VMEM>
__device__ __forceinline__ void schedule_phase() {
  if constexpr (M < MFMAS) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (M < DSR) __builtin_amdgcn_sched_group_barrier(0x100, 1 + (M == 0 ? (DSR > MFMAS ? DSR - MFMAS : 0) : 0), 0);
    if constexpr (VALU > 0) __builtin_amdgcn_sched_group_barrier(0x002, (VALU + MFMAS - 1) / MFMAS, 0);
    if constexpr (DSW > 0) __builtin_amdgcn_sched_group_barrier(0x200, (DSW + MFMAS - 1) / MFMAS, 0);
    if constexpr (VMEM > 0) __builtin_amdgcn_sched_group_barrier(0x020, (VMEM + MFMAS - 1) / MFMAS, 0);
    schedule_phase<M + 1, MFMAS, DSR, DSW, VALU, VMEM>();
  }
}

// One grouped-GEMM kernel, templated on the weight format, on whether two banks (gate, up) are multiplied in
// the same launch with the SwiGLU epilogue, and on the block tile: BM rows x BN columns of each matrix. The
// four wavefronts sit WM x WN (1 x 4: side by side along the columns, so no two of them need the same weight
// bytes); each owns (BM/WM) x (BN/WN) of every matrix as 32 x 32 MFMA tiles.
template <int FORMAT, int MODE, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(kThreads, (FORMAT != DEW_MOE_W_BF16 && BM == 128 && ((MODE == kSwigluOfTwo || MODE == kSwigluOfTwoSplit) ? 2 : 1) * BN == 256) ? 2 : 1) void grouped_gemm_kernel(GemmParams p) {
  constexpr bool PAIRED = MODE == kSwigluOfTwo || MODE == kSwigluOfTwoSplit;
  constexpr bool kSplitOut = MODE == kSwigluOfTwoSplit;
  // Unquantized and FP4 banks (their atoms are 64 deep and 32 columns wide at most) take a depth in whole 64-deep steps and a
  // width in whole 32-column atoms, close to the multiples of 8 of the reference's own grouped kernel: a strip past the width
  // multiplies columns it does not store. (GPT-OSS's experts are 2880 wide: 45 steps, 90 atoms, no whole 128s.)
  constexpr bool kNvF16 = FORMAT == kFormatNvF16;  // f16 rows under a scale a row, a general NVFP4 bank decoded to f16
  static_assert(!kNvF16 || MODE == kSwigluOfTwo, "f16 rows: the paired launch");
  constexpr bool kRagged = FORMAT == DEW_MOE_W_BF16 || FORMAT == DEW_MOE_W_MXFP4 || FORMAT == DEW_MOE_W_NVFP4 || kNvF16;
  constexpr bool kGated = MODE == kInterleavedGated;
  constexpr int kOutBN = kGated ? BN / 2 : BN;  // output columns of the tile
  static_assert(WM * WN == 4 && BM % (32 * WM) == 0 && BN % (32 * WN) == 0 && BM % 32 == 0, "tile shape");
  constexpr bool kFp8Rows = FORMAT == kFormatFp8Rows;   // e4m3 rows, one scale per row and 128 depths; 128 x 128 weight scales
  constexpr bool kWindow = FORMAT == kFormatMxFp8Window || FORMAT == kFormatBf16Window;  // a kernel gradient: the same rows for every group, its own depths
  constexpr bool kMxRows = FORMAT == kFormatMxFp8Rows || FORMAT == kFormatMxFp8Window;  // e4m3 rows and weights, one scale per row (column) and 32 depths
  constexpr bool kFp8A = kFp8Rows || kMxRows;           // both operands e4m3 codes: a step is 128 depths
  constexpr bool kHi6 = FORMAT == kFormatMxSplit66;     // both terms of a row in FP6 (e2m3), each with its scale beside it
  constexpr bool kLo6 = FORMAT == kFormatMxSplit6 || kHi6;  // the second term of a row in FP6 (e2m3), its scale beside it
  constexpr bool kSplit = FORMAT == kFormatMxSplit || FORMAT == kFormatMxSplitBlocks || kLo6 || kFp8A;  // A arrives as 8-bit codes
  constexpr bool kBlockScales = FORMAT == kFormatMxSplitBlocks || kFp8Rows;
  constexpr bool kFp4 = FORMAT == DEW_MOE_W_NVFP4 || FORMAT == DEW_MOE_W_MXFP4 || kNvF16 || (kSplit && !kFp8A);
  constexpr bool kPow2 = FORMAT == DEW_MOE_W_MXFP4 || (kSplit && !kFp8A);
  constexpr bool kBlockBank = FORMAT == DEW_MOE_W_FP8_BLOCK || kFp8Rows;  // one fp32 scale per 128 x 128 weights
  constexpr int kMatrices = PAIRED ? 2 : 1;
  constexpr bool kBf16 = FORMAT == DEW_MOE_W_BF16 || FORMAT == kFormatBf16Window;  // unquantized matrices: the atoms are the fragments themselves
  constexpr int kAtomK = kFp4 ? 64 : kBf16 ? 16 : 32;  // depth an atom covers
  constexpr int kStepDepth = kFp8A ? 128 : BK;  // depth a step covers: always 128 bytes of an A row
  constexpr int kAtoms = kStepDepth / kAtomK;  // 16-byte loads a lane makes per 32-column tile per step
  constexpr int kRowLoads = BM / 32;           // A rows a lane loads per step
  constexpr int TI = BM / (32 * WM), TJ = BN / (32 * WN);  // MFMA tiles per wavefront: rows, columns of each matrix
  constexpr int kTiles = kMatrices * TJ;       // weight tiles a wavefront multiplies
  constexpr int kStageChunks = BM * kChunksPerRow;
  constexpr int kStages = 3;
  // Weight register sets in flight. The 128-row tile of 256 columns in all (paired 2 x 128, or unpaired 256: two
  // MFMAs for each A fragment read from LDS) runs two blocks a CU (256 registers a lane each),
  // which FP8's 32 raw bytes a lane a tile a step only fit with three sets; two resident blocks cover the
  // shorter lookahead.
  // Quantized rows on the full 256 x 256 tile: a step's weights are 64 registers a lane, of which two sets fit
  // beside the accumulators (a load then has most of a 2048-cycle step to land).
  // (bf16 matrices: a step's raw data is twice FP8's, three sets of it fit beside the 256-row tile's accumulators)
  constexpr int kSets = (kFp8A && BN == 256) ? 2 : (kSplit && !kFp8A && BM == 128) ? 2 : (kBf16 || (!kFp4 && BM == 128 && kMatrices * BN == 256)) ? 3 : 4;

  extern __shared__ u32x4_t lds[];  // a ring of three stages of A: BM rows of 128 bytes each
  __shared__ int wave_tiles[4], wave_rows[4];
  __shared__ int found[5];  // expert, first sorted row of the tile, total m-tiles, the expert's last row + 1, rows in all groups
  // FP8 128 x 128 blocks: the scales of the block's column blocks down the whole depth, read once
  constexpr int kScaleColumns = kBlockBank ? kMatrices * (BN / 128) : 1;
  __shared__ float depth_scales[kScaleColumns][kBlockBank ? kMaxDepthBlocks : 1];

  __shared__ float row_factor[kNvF16 ? BM : 1];  // f16 rows: 2^s of each of the tile's rows, which its sums are owed

  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;

  // ---- block -> (m-tile, column strip). Workgroup ids are dealt round-robin to the 8 XCDs, each with its
  // own L2. Tiles are ordered so that a chunk of consecutive ones (one XCD's residents) covers kGroupM m-tiles x 8
  // strips, sharing A rows and B strips through that L2, and such chunks of 32 are dealt round-robin to the
  // XCDs: the m-tile bound overshoots the real tile count by up to one tile per expert, and the empty tiles
  // at the end of the order then spread over all XCDs instead of idling the last ones.
  const int kGroupM = p.group_m, kChunk = 8 * kGroupM;
  // (a bf16 bank's width need not be whole strips: its last strip then holds fewer columns than BN, see kRagged below)
  const int n_strips = (p.width + BN - 1) / BN;
  const int total = p.m_tile_bound * n_strips;
  const int local = blockIdx.x / 8;
  const int order = ((local / kChunk) * 8 + blockIdx.x % 8) * kChunk + local % kChunk;
  if (order >= total) return;
  const int group = order / (kGroupM * n_strips);
  const int group_m = min(kGroupM, p.m_tile_bound - group * kGroupM);
  const int within = order % (kGroupM * n_strips);
  const int m_tile = group * kGroupM + within % group_m;
  const int n0 = (within / group_m) * BN;

  // ---- which expert owns m-tile `m_tile`? inclusive scan of ceil(size / BM) over the experts (and, where the caller
  // gave group sizes instead of their prefix, of the sizes themselves: an expert's first row) ----
  if (tid == 0) found[0] = -1;
  int carried = 0, carried_rows = 0;
  // (a round's sizes and first rows are asked for one round ahead: past 256 experts the rounds' loads then overlap, instead
  // of one memory round trip a round in front of every tile)
  auto size_of = [&](int e) { return e >= p.experts ? 0 : kWindow ? p.window_rows : p.sizes ? max(p.sizes[e], 0) : p.offsets[e + 1] - p.offsets[e]; };
  auto first_row_of = [&](int e) { return e >= p.experts || (p.sizes && !kWindow) ? 0 : kWindow ? e * p.window_rows : p.offsets[e]; };
  int next_size = size_of(tid), next_first_row = first_row_of(tid);
  for (int base = 0; base < p.experts; base += kThreads) {
    const int e = base + tid;
    int start = 0, tiles = 0;
    const int size = next_size, first_row = next_first_row;
    next_size = size_of(e + kThreads);
    next_first_row = first_row_of(e + kThreads);
    if (p.sizes && !kWindow) {  // (uniform) exclusive prefix of the sizes
      int inclusive_rows = size;
#pragma unroll
      for (int offset = 1; offset < 64; offset <<= 1) {
        const int other = __shfl_up(inclusive_rows, offset, 64);
        if (lane >= offset) inclusive_rows += other;
      }
      __syncthreads();
      if (lane == 63) wave_rows[wave] = inclusive_rows;
      __syncthreads();
      start = carried_rows + inclusive_rows - size;
      for (int w = 0; w < wave; ++w) start += wave_rows[w];
      carried_rows += wave_rows[0] + wave_rows[1] + wave_rows[2] + wave_rows[3];
    } else {
      start = first_row;
    }
    const int group_end = start + size;
    if (e < p.experts) {
      if (p.tail_of > 0) {
        const int rest = size % p.tail_of;
        tiles = rest >= 1 && rest <= BM ? 1 : 0;
        start += size - rest;
      } else {
        tiles = size / BM + (size % BM > p.skip_tails ? 1 : 0);
      }
    }
    int inclusive = tiles;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const int other = __shfl_up(inclusive, offset, 64);
      if (lane >= offset) inclusive += other;
    }
    __syncthreads();
    if (lane == 63) wave_tiles[wave] = inclusive;
    __syncthreads();
    int before = carried;
    for (int w = 0; w < wave; ++w) before += wave_tiles[w];
    const int first = before + inclusive - tiles;
    if (tiles > 0 && m_tile >= first && m_tile < first + tiles) {
      found[0] = e;
      found[1] = start + (m_tile - first) * BM;
      found[3] = group_end;
    }
    carried += wave_tiles[0] + wave_tiles[1] + wave_tiles[2] + wave_tiles[3];
  }
  if (tid == 0) {
    found[2] = carried;
    found[4] = p.sizes ? carried_rows : 0;  // the rows the groups hold (read from the prefix's last entry otherwise)
  }
  __syncthreads();
  const int expert = found[0];

  if (expert < 0) {
    if (kWindow || p.tail_of > 0) return;  // (the taller tiles' launch zeroes them; a kernel gradient has no rows past its groups)
    // Past the last real tile: zero the rows no expert owns (sorted positions offsets[E] .. rows).
    const int tail_begin = (p.sizes ? found[4] : p.offsets[p.experts]) + (m_tile - found[2]) * BM;
    const int tail_end = min(tail_begin + BM, p.rows);
    const int out_width = kGated ? p.width / 2 : p.width, out_n0 = kGated ? n0 / 2 : n0;
    for (int item = tid; item < (tail_end - tail_begin) * (kOutBN / 8); item += kThreads) {
      const int sorted = tail_begin + item / (kOutBN / 8);
      const int row = p.scatter ? p.scatter[sorted] : sorted;
      if (kRagged && out_n0 + (item % (kOutBN / 8)) * 8 >= out_width) continue;  // the last strip's columns past the width
      *reinterpret_cast<u32x4_t*>(p.out + static_cast<size_t>(row) * out_width + out_n0 + (item % (kOutBN / 8)) * 8) = u32x4_t{0, 0, 0, 0};
      if constexpr (kSplitOut) {  // zero terms under a unit scale
        if (item % (kOutBN / 8) == 0) p.out_scale[static_cast<size_t>(sorted) * block_scale_pitch(p.width) + n0 / 128] = 127;
      }
    }
    return;
  }

  const int row0 = found[1];
  const int valid_rows = min(BM, found[3] - row0);
  // a kernel gradient's group contracts its own whole steps of the depth (128 tokens of e4m3 codes, 64 of bf16)
  const int first_step = kWindow ? min(max(p.windows[expert], 0), p.depth) / kStepDepth : 0;
  const int steps = kWindow ? max(min(max(p.windows[expert + 1], 0), p.depth) / kStepDepth - first_step, 0) : p.depth / kStepDepth;
  if (kWindow && steps == 0) {  // an empty group's gradient is zero
    for (int item = tid; item < valid_rows * (BN / 4); item += kThreads) {
      const size_t at = static_cast<size_t>(row0 + item / (BN / 4)) * p.width + n0 + (item % (BN / 4)) * 4;
      if (MODE == kPlainF32)
        *reinterpret_cast<u32x4_t*>(p.out_f32 + at) = u32x4_t{0, 0, 0, 0};
      else
        *reinterpret_cast<uint2*>(p.out + at) = uint2{0, 0};
    }
    return;
  }
  const int wm0 = (wave / WN) * (BM / WM), wn0 = (wave % WN) * (BN / WN);

  // ---- B loader: tile t = (matrix, 32-column tile j of the wavefront); the lane's piece of each atom ----
  const uint8_t* b_src[kTiles];
  const uint8_t* b_scale_src[kTiles];  // FP4: the lane's two e4m3 block scales of each atom
  float channel_scale[kTiles];         // FP8 channel: the lane's column scale
  const int n_atoms = p.width / 32, k_atoms = p.depth / kAtomK;
  const uint32_t b_lane = lane * 16, b_scale_lane = lane * 2;
#pragma unroll
  for (int t = 0; t < kTiles; ++t) {
    // (past a ragged width the tile reads the bank's last 32 columns again, inside the expert's matrix; its results are not stored)
    const int matrix = t / TJ, column = kRagged ? min(n0 + wn0 + 32 * (t % TJ), p.width - 32) : n0 + wn0 + 32 * (t % TJ);
    const uint8_t* codes = matrix == 0 ? p.w0.codes : p.w1.codes;
    const void* scales = matrix == 0 ? p.w0.scales : p.w1.scales;
    // (a kernel gradient's one "expert" holds every group's tokens: the group's window starts first_step steps in)
    const size_t first_atom = (static_cast<size_t>(kWindow ? 0 : expert) * n_atoms + column / 32) * k_atoms + first_step * kAtoms;
    b_src[t] = codes + first_atom * kAtomBytes + b_lane;
    b_scale_src[t] = nullptr;
    channel_scale[t] = 1.0f;
    if (kFp4) {
      b_scale_src[t] = static_cast<const uint8_t*>(scales) + first_atom * 128 + b_scale_lane;
    } else if (kMxRows) {  // [E][N / 32][K / 128][32 columns][4 bytes]: the lane's column's dword of each step
      b_scale_src[t] = static_cast<const uint8_t*>(scales) +
                       ((static_cast<size_t>(kWindow ? 0 : expert) * n_atoms + column / 32) * (p.depth / 128) + first_step) * 128 + (lane % 32) * 4;
    } else if (FORMAT == DEW_MOE_W_FP8_CHANNEL) {
      channel_scale[t] = static_cast<const float*>(scales)[static_cast<size_t>(expert) * p.width + column + lane % 32];
    }
  }
  // FP8 128 x 128 blocks: this thread's first block scale goes into a register now, ahead of the weight loads, and into
  // the LDS table further down, once the loads behind it are out (a launch of at most 256 scale entries a tile, every
  // one but the deepest, has no other; the rest are copied there in a loop).
  float early_scale = 0.0f;
  if constexpr (kBlockBank) {
    const int depth_blocks = p.depth / 128, width_blocks = p.width / 128;
    if (tid < kScaleColumns * depth_blocks) {
      const int which = tid / depth_blocks, block = tid % depth_blocks;
      const float* scales = static_cast<const float*>(which / (BN / 128) == 0 ? p.w0.scales : p.w1.scales);
      early_scale = scales[(static_cast<size_t>(expert) * depth_blocks + block) * width_blocks + n0 / 128 + which % (BN / 128)];
    }
  }

  // FP4 banks: the expert's tensor scales, which the epilogue multiplies by, are asked for here as well (fetched there, the
  // epilogue's arithmetic began with a memory round trip)
  float tensor_scale0 = 1.0f, tensor_scale1 = 1.0f;
  if constexpr (kFp4) {
    tensor_scale0 = p.w0.tensor_scale[expert];
    if constexpr (PAIRED) tensor_scale1 = p.w1.tensor_scale[expert];
  }

  // Raw weight data in flight: kSets register sets (steps s .. s + kSets - 1), so a load has kSets - 2 to
  // kSets - 1 steps to land.
  u32x4_t b_regs[kSets][kTiles][kAtoms];
  uint32_t s_regs[kSets][kTiles];  // FP4: two e4m3 scale bytes in the low half
  auto load_b = [&](auto set, int step, auto begin, auto end) __attribute__((always_inline)) {
#pragma unroll
    for (int t = begin.value; t < end.value; ++t) {
#pragma unroll
      for (int a = 0; a < kAtoms; ++a) {
        const u32x4_t* from = reinterpret_cast<const u32x4_t*>(b_src[t] + (static_cast<size_t>(step) * kAtoms + a) * kAtomBytes);
        // Decode-sized groups (the 32-row tiles) read every weight byte once: loaded as non-temporal the stream runs 3 to 6 %
        // faster (a read-only stream of 16-byte loads measures 7.1 TB/s so hinted against 5.6 to 6.4 without). Taller
        // tiles keep the plain load: their groups' tiles share weight strips through the L2 (128-row tiles: 2 to 4 % slower
        // with the hint).
        if constexpr (BM <= 32)
          b_regs[set.value][t][a] = __builtin_nontemporal_load(from);
        else
          b_regs[set.value][t][a] = *from;
      }
      if constexpr (kMxRows) {  // a dword a lane: its column's four scale bytes of the step
        __builtin_memcpy(&s_regs[set.value][t], b_scale_src[t] + static_cast<size_t>(step) * 128, sizeof(uint32_t));
      } else if constexpr (kFp4) {
        // the lane's two e4m3 bytes as the aligned 16-bit load they are (a dword load at 2 lane is misaligned in every
        // other lane and reads two bytes past the lane's own: 2.4 % of the split-row paired launch)
        s_regs[set.value][t] = *reinterpret_cast<const uint16_t*>(b_scale_src[t] + static_cast<size_t>(step) * 128);
      }
    }
  };

  // A tile's start is a chain of dependent loads: the groups' offsets, then the rows' gather indices, then the rows and
  // their scales. The weights depend on the first link alone. So the gather indices are asked for first and the first
  // weight loads right behind them, before anything waits: loads return in order, the indices are back after one round
  // trip with the weights still in flight, and the rows' loads follow them. (Issued behind the other set-up, as they
  // were, the weights started two round trips later: about 1.5 us of a decode launch's 35 to 70.)
  int a_source[kRowLoads];  // the source row of each of this lane's row loads
#pragma unroll
  for (int i = 0; i < kRowLoads; ++i) {
    const int sorted = row0 + min((wave * kRowLoads + i) * 8 + lane / 8, valid_rows - 1);
    a_source[i] = kWindow ? sorted - expert * p.window_rows : p.gather ? p.gather[sorted] : sorted;
  }
  int tile_source[kSplit ? TI : 1];  // split rows: the lane's row of each row tile
  if constexpr (kSplit) {
#pragma unroll
    for (int i = 0; i < TI; ++i) {
      const int sorted = row0 + min(wm0 + 32 * i + lane % 32, valid_rows - 1);
      tile_source[i] = p.gather ? p.gather[sorted] : sorted;
    }
  }
  int thread_source = 0;  // row tid of the tile, where one thread fetches one row's scales
  if constexpr (kNvF16 || kBlockScales || kMxRows) {
    if (tid < BM) {
      const int sorted = row0 + min(tid, valid_rows - 1);
      thread_source = kWindow ? sorted - expert * p.window_rows : p.gather ? p.gather[sorted] : sorted;
    }
  }
  {
    constexpr std::integral_constant<int, 0> set0{};
    constexpr std::integral_constant<int, 1> set1{};
    constexpr std::integral_constant<int, 2> set2{};
    constexpr std::integral_constant<int, kTiles> every_tile{};
    load_b(set0, 0, set0, every_tile);
    if constexpr (kSets >= 3) load_b(set1, min(1, steps - 1), set0, every_tile);
    if constexpr (kSets == 4) load_b(set2, min(2, steps - 1), set0, every_tile);
  }

  if constexpr (kNvF16) {
    static_assert(!kNvF16 || BM <= kThreads, "one thread fetches one row's scale");
    if (tid < BM)  // (read in the epilogue, behind the loop's barriers)
      row_factor[tid] = __uint_as_float(static_cast<uint32_t>(p.a_scale[thread_source]) << 23);
  }

  // ---- A loader. One global_load_lds_dwordx4 of a wavefront fills 1 KiB of LDS, lane l landing at byte 16 l:
  // 8 rows of a stage, lane l = row l / 8, stored chunk l % 8. The lane therefore fetches the logical chunk
  // that the swizzle keeps at that place. Wavefront w issues the loads of rows 8 (w kRowLoads + i) .. + 7.
  const bf16_t* a_src[kRowLoads];
#pragma unroll
  for (int i = 0; i < kRowLoads; ++i) {
    const int row = (wave * kRowLoads + i) * 8 + lane / 8;
    const int chunk = (lane % 8) ^ (((row >> 1) & 7) ^ ((row & 1) << 2));
    // (a row of e4m3 codes is depth bytes.) Less the load's immediate offset, which the instruction adds back: see load_a
    a_src[i] = p.x + static_cast<size_t>(a_source[i]) * (kFp8A ? p.depth / 2 : p.depth) + first_step * (kFp8A ? kStepDepth / 2 : kStepDepth) + chunk * 8 - (i % 4) * 512;
    asm volatile("" : "+v"(a_src[i]));  // kept as computed: the compiler otherwise re-adds the bias at every load
  }
  // Split activations: the lane's row of each row tile carries one e8m0 scale; the hi term multiplies under it
  // (byte 0) and the lo term under 2^-4 of it (byte 1).
  int a_scale_word[TI];
#pragma unroll
  for (int i = 0; i < TI; ++i) {
    a_scale_word[i] = 0;
    if constexpr (kSplit) {
      if constexpr (!kBlockScales && !kHi6) {  // (two FP6 terms carry their scales with their codes)
        const int byte = p.a_scale[tile_source[i]];
        a_scale_word[i] = byte | ((byte - 4) << 8);
      }
    }
  }
  // Block scales change every 128 depths (two steps). The tile's rows' scales, all depths of them, are copied into
  // the LDS behind the ring before the loop (thread t copies row t, 16 bytes a load), and the loop reads its bytes
  // from there into two sets of registers, the one of the next 128 depths while this one multiplies. (Read from
  // global memory inside the loop they cost 14 to 20 % of the kernel, however early they were issued: every byte
  // is a first touch of its cache line, and the vmcnt wait of each step's barrier, which counts loads in order,
  // stalled on them.)
  const int a_pitch = block_scale_pitch(p.depth);
  uint8_t* block_scales = reinterpret_cast<uint8_t*>(lds + kStages * kStageChunks);
  if constexpr (kBlockScales) {
    static_assert(!kBlockScales || BM <= kThreads, "one thread copies one row's scales");
    if (tid < BM) {
      const u32x4_t* from = reinterpret_cast<const u32x4_t*>(p.a_scale + static_cast<size_t>(thread_source) * a_pitch);
      u32x4_t* to = reinterpret_cast<u32x4_t*>(block_scales + tid * a_pitch);
      for (int piece = 0; piece < a_pitch / 16; ++piece) to[piece] = from[piece];
    }
  }
  int a_block_word[2][kBlockScales ? TI : 1], a_block_byte[kBlockScales ? TI : 1];
  auto load_block_scales = [&](int block) __attribute__((always_inline)) {
    if constexpr (kBlockScales) {
#pragma unroll
      for (int i = 0; i < TI; ++i) a_block_byte[i] = block_scales[(wm0 + 32 * i + lane % 32) * a_pitch + block];
    }
  };
  auto form_block_words = [&](auto buffer) __attribute__((always_inline)) {
    if constexpr (kBlockScales) {
#pragma unroll
      for (int i = 0; i < TI; ++i)  // quantized rows have the one term: the byte is the word
        a_block_word[buffer.value][i] = kFp8Rows ? a_block_byte[i] : a_block_byte[i] | ((a_block_byte[i] - 4) << 8);
    }
  };
  // The LDS address of such a load is M0 + its immediate offset + 16 lane, and M0 costs three instructions to set
  // (a lane read, the move, a wait state): four loads share one M0, the base of their first, and reach their own
  // KiB of the stage through the immediate offset, which the global address is biased against (a_src above).
  auto load_a = [&](u32x4_t* stage, int step, auto begin, auto end) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass, which only needs the kernel's stub, does not know the builtin
    static_range<decltype(begin)::value>(std::make_integer_sequence<int, decltype(end)::value - decltype(begin)::value>{}, [&](auto index) {
      constexpr int i = decltype(index)::value, first = i / 4 * 4;
      __builtin_amdgcn_global_load_lds(a_src[i] + static_cast<size_t>(step) * BK,
                                       (__attribute__((address_space(3))) void*)(stage + (wave * kRowLoads + first) * 64), 16,
                                       (i - first) * 1024, 0);
    });
#endif
  };

  // MXFP8 rows: a step's four scale bytes of each row, one dword a row, ride the ring beside the A rows: thread t
  // fetches row t's (one 4-byte LDS-DMA load a wavefront a step), into BM dwords a stage behind the ring.
  uint32_t* a_mx_stage = reinterpret_cast<uint32_t*>(lds + kStages * kStageChunks);
  const uint8_t* a_mx_src = nullptr;
  (void)a_mx_src;  // (the host pass compiles no load)
  if constexpr (kMxRows) {
    static_assert(!kMxRows || BM == kThreads, "one thread fetches one row's scales");
    a_mx_src = p.a_scale + static_cast<size_t>(thread_source) * (p.depth / 32) + first_step * 4;
  }
  auto load_a_scales = [&](int stage_number, int step) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (kMxRows)
      __builtin_amdgcn_global_load_lds(a_mx_src + 4 * step, (__attribute__((address_space(3))) void*)(a_mx_stage + stage_number * BM + wave * 64),
                                       4, 0, 0);
#endif
  };
  uint32_t a_mx_word[2][kMxRows ? TI : 1];  // the lane's rows' scale dwords of a step, shifted so that byte 2 t is term t's
  auto fetch_a_scales = [&](auto buffer, int stage_number) __attribute__((always_inline)) {
    if constexpr (kMxRows) {
#pragma unroll
      for (int i = 0; i < TI; ++i)
        a_mx_word[buffer.value][i] = a_mx_stage[stage_number * BM + wm0 + 32 * i + lane % 32] >> (8 * (lane / 32));
    }
  };

  if constexpr (kBlockBank) {
    const int depth_blocks = p.depth / 128, width_blocks = p.width / 128;
    if (tid < kScaleColumns * depth_blocks) depth_scales[tid / depth_blocks][tid % depth_blocks] = early_scale;
    for (int item = tid + kThreads; item < kScaleColumns * depth_blocks; item += kThreads) {
      const int which = item / depth_blocks, block = item % depth_blocks;
      const float* scales = static_cast<const float*>(which / (BN / 128) == 0 ? p.w0.scales : p.w1.scales);
      depth_scales[which][block] =
          scales[(static_cast<size_t>(expert) * depth_blocks + block) * width_blocks + n0 / 128 + which % (BN / 128)];
    }
  }

  // ---- fragments: slice kk of a step is 16 depths; a lane's are the 8 its weight bytes cover ----
  bf16x8_t a_frag[2][TI], b_frag[2][kTiles];
  i32x8_t a_term[2][kSplit ? TI : 1];  // split activations: [0] the hi term of a step, [1] its lo term
  int a_fp6_scale[2][kLo6 ? TI : 1];   // an FP6 term's e8m0 scale of the lane's 32 depths (it lies behind the codes)
  float fp4_scale[kTiles];
  _Float16 fp4_half[kNvF16 ? kTiles : 1];  // f16 rows: the block scale as f16
  // a term of a 32-depth block is 32 bytes: the lane's block lane / 32 of the step holds hi in its chunks 0-1, lo in 2-3
  // The lane's four chunks of its first row tile, as chunk indices into a stage: computed once, so that a phase's
  // reads are the stage's base plus one of these plus 32 rows (a constant) a row tile further.
  int term_chunk[2][2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int piece = 0; piece < 2; ++piece) term_chunk[t][piece] = swizzled(wm0 + lane % 32, 4 * (lane / 32) + 2 * t + piece);
  auto fetch_term = [&](const u32x4_t* stage, auto term) __attribute__((always_inline)) {
    if constexpr (kSplit) {
      const u32x4_t* first_piece = stage + term_chunk[term.value][0];
      const u32x4_t* second_piece = stage + term_chunk[term.value][1];
#pragma unroll
      for (int i = 0; i < TI; ++i) {
        const u32x4_t first = first_piece[32 * i * kChunksPerRow];  // the swizzle reads a row's low four bits only
        const u32x4_t second = second_piece[32 * i * kChunksPerRow];
        if constexpr ((kLo6 && term.value == 1) || kHi6) {  // 24 bytes of e2m3 codes, then the scale's dword
          a_term[term.value][i] = i32x8_t{static_cast<int>(first[0]), static_cast<int>(first[1]), static_cast<int>(first[2]),
                                          static_cast<int>(first[3]), static_cast<int>(second[0]), static_cast<int>(second[1]), 0, 0};
          a_fp6_scale[term.value][i] = static_cast<int>(second[2]);
        } else {
          a_term[term.value][i] = i32x8_t{static_cast<int>(first[0]), static_cast<int>(first[1]), static_cast<int>(first[2]),
                                          static_cast<int>(first[3]), static_cast<int>(second[0]), static_cast<int>(second[1]),
                                          static_cast<int>(second[2]), static_cast<int>(second[3])};
        }
      }
    }
  };
  auto fetch = [&](const u32x4_t* stage, auto kk, auto into) __attribute__((always_inline)) {
    const int chunk = kFp4 ? 4 * (lane / 32) + kk.value : kBf16 ? 2 * kk.value + lane / 32 : 4 * (kk.value / 2) + 2 * (lane / 32) + kk.value % 2;
#pragma unroll
    for (int i = 0; i < TI; ++i)
      a_frag[into.value][i] = __builtin_bit_cast(bf16x8_t, stage[swizzled(wm0 + 32 * i + lane % 32, chunk)]);
  };
  auto dequantize = [&](auto set, auto kk, auto into, int step) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < kTiles; ++t) {
      if constexpr (kNvF16) {
        if constexpr (kk.value % 2 == 0)  // slices 0, 1 lie in the lane's first 16-deep block, 2, 3 in its second
          fp4_half[t] = static_cast<_Float16>(kk.value == 0 ? __builtin_amdgcn_cvt_f32_fp8(s_regs[set.value][t], 0)
                                                            : __builtin_amdgcn_cvt_f32_fp8(s_regs[set.value][t], 1));
        b_frag[into.value][t] = fragment_fp4_f16(b_regs[set.value][t][0][kk.value], fp4_half[t]);
      } else if constexpr (kFp4) {
        if constexpr (kk.value % 2 == 0)  // slices 0, 1 lie in the lane's first 16-deep block, 2, 3 in its second
          fp4_scale[t] = (kk.value == 0 ? __builtin_amdgcn_cvt_f32_fp8(s_regs[set.value][t], 0)
                                        : __builtin_amdgcn_cvt_f32_fp8(s_regs[set.value][t], 1)) * 0.00390625f;
        const uint32_t word = b_regs[set.value][t][0][kk.value];
        b_frag[into.value][t] = kPow2 ? fragment_fp4_pow2(word, fp4_scale[t]) : fragment_fp4(word, fp4_scale[t]);
      } else if constexpr (kBf16) {
        b_frag[into.value][t] = __builtin_bit_cast(bf16x8_t, b_regs[set.value][t][kk.value]);
      } else {
        const float scale = FORMAT == DEW_MOE_W_FP8_BLOCK
                                ? depth_scales[(t / TJ) * (BN / 128) + (wn0 + 32 * (t % TJ)) / 128][step / (128 / BK)]
                                : channel_scale[t];
        const u32x4_t& raw = b_regs[set.value][t][kk.value / 2 % kAtoms];
        b_frag[into.value][t] = fragment_fp8(raw[2 * (kk.value % 2)], raw[2 * (kk.value % 2) + 1], scale);
      }
    }
  };

  f32x16_t acc[kMatrices][TI][TJ];
#pragma unroll
  for (int m = 0; m < kMatrices; ++m)
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int j = 0; j < TJ; ++j)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[m][i][j][q] = 0.0f;
  auto multiply = [&](auto from) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < kMatrices; ++m)
#pragma unroll
      for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
          if constexpr (kNvF16)
            acc[m][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a_frag[from.value][i]),
                                                                  __builtin_bit_cast(f16x8_t, b_frag[from.value][m * TJ + j]), acc[m][i][j], 0, 0, 0);
          else
            acc[m][i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_frag[from.value][i], b_frag[from.value][m * TJ + j], acc[m][i][j], 0, 0, 0);
        }
  };

  // Split activations: one scaled instruction multiplies 64 depths of one term by the stored FP4 codes under
  // both operands' power-of-two scales; the block scale byte is the e4m3 of a normal power of two, 2^(field - 7).
  int unscalable = 0;  // quantized rows: mantissa bits met in a weight block scale (the instruction takes powers of two only)
  auto multiply_term = [&](auto set, auto term, int step, auto buffer) __attribute__((always_inline)) {
    if constexpr (kSplit) {
      // block scales: of the unrolled four steps, steps 0, 1 read buffer 0 and steps 2, 3 buffer 1 (a scale holds for
      // two 64-deep steps); quantized rows' 128-deep steps alternate
      constexpr int kBuffer = buffer.value;
#pragma unroll
      for (int m = 0; m < kMatrices; ++m)
#pragma unroll
        for (int j = 0; j < TJ; ++j) {
          if constexpr (kFp8A) {
            // both operands e4m3: the half's 64 depths are two 32-deep atoms of the bank, in the operand's own order
            const u32x4_t& first = b_regs[set.value][m * TJ + j][2 * term.value];
            const u32x4_t& second = b_regs[set.value][m * TJ + j][2 * term.value + 1];
            const i32x8_t codes = {static_cast<int>(first[0]), static_cast<int>(first[1]), static_cast<int>(first[2]), static_cast<int>(first[3]),
                                   static_cast<int>(second[0]), static_cast<int>(second[1]), static_cast<int>(second[2]), static_cast<int>(second[3])};
            if constexpr (kMxRows) {
              // each lane hands in the scale of its row (column) and its lane group's 32 of the half's 64 depths:
              // byte 2 term + lane / 32 of the step's dword, brought to byte 2 term by the shift
              const int b_scale = static_cast<int>(s_regs[set.value][m * TJ + j] >> (8 * (lane / 32)));
#pragma unroll
              for (int i = 0; i < TI; ++i)
                acc[m][i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_term[term.value][i], codes, acc[m][i][j], 0, 0, 2 * term.value,
                                                                            static_cast<int>(a_mx_word[kBuffer][i]), 2 * term.value, b_scale);
            } else {
              const uint32_t bits = __float_as_uint(depth_scales[m * (BN / 128) + (wn0 + 32 * j) / 128][step]);
              unscalable |= (bits & 0x807FFFFFu) | ((bits >> 23) == 0u) | ((bits >> 23) == 255u);
              const int b_scale = static_cast<int>(bits >> 23);
#pragma unroll
              for (int i = 0; i < TI; ++i)
                acc[m][i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_term[term.value][i], codes, acc[m][i][j], 0, 0, 0,
                                                                            a_block_word[kBuffer][i], 0, b_scale);
            }
          } else {
            const u32x4_t& raw = b_regs[set.value][m * TJ + j][0];
            const i32x8_t codes = {static_cast<int>(raw[0]), static_cast<int>(raw[1]), static_cast<int>(raw[2]), static_cast<int>(raw[3]), 0, 0, 0, 0};
            const int b_scale = static_cast<int>(((s_regs[set.value][m * TJ + j] >> 3) & 15u) + 120u);
#pragma unroll
            for (int i = 0; i < TI; ++i) {
              if constexpr ((kLo6 && term.value == 1) || kHi6) {  // FP6 (e2m3) x FP4 under the term's own scale
                acc[m][i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_term[term.value][i], codes, acc[m][i][j], 2, 4, 0,
                                                                            a_fp6_scale[term.value][i], 0, b_scale);
              } else {
                acc[m][i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a_term[term.value][i], codes, acc[m][i][j], 0, 4, term.value,
                                                                            kBlockScales ? a_block_word[kBuffer][i] : a_scale_word[i], 0,
                                                                            b_scale);
              }
            }
          }
        }
    }
  };

  // ---- pipeline. At the top of step s: LDS stage s % 3 holds the A rows of step s and the loads of step s + 1
  // into stage (s + 1) % 3 are in flight; B register sets s % 4 .. (s + 2) % 4 hold (or are receiving) steps
  // s .. s + 2. A step is four phases, one 16-deep slice each: the slice multiplies while the next slice's A
  // fragments are read from LDS and its B fragments dequantized. Each phase also issues a quarter of the step's
  // global loads, so the memory pipeline sees an even stream: A rows of step s + 2 into stage (s + 2) % 3 (last
  // read during step s - 1) and weights of step s + kSets - 1 into the set last read during step s - 1.
  // One barrier a step, after phase 3: by then this wavefront's A loads of step s + 1 have landed (a vmcnt wait
  // that leaves the younger loads in flight) and its own fragment reads are done, so after the barrier stage
  // (s + 1) % 3 may be read and stage s % 3 overwritten. The loop is unrolled by kSets so that the B register
  // sets are compile-time constants.
  constexpr std::integral_constant<int, 0> c0{};
  constexpr std::integral_constant<int, 1> c1{};
  constexpr std::integral_constant<int, 2> c2{};
  constexpr std::integral_constant<int, 3> c3{};
  constexpr std::integral_constant<int, (kRowLoads + 3) / 4> a1{};  // A loads early in the step, weights late
  constexpr std::integral_constant<int, (2 * kRowLoads + 3) / 4> a2{};
  constexpr std::integral_constant<int, (3 * kRowLoads + 3) / 4> a3{};
  constexpr std::integral_constant<int, kRowLoads> a4{};
  constexpr std::integral_constant<int, kTiles / 4> b1{};
  constexpr std::integral_constant<int, 2 * kTiles / 4> b2{};
  constexpr std::integral_constant<int, 3 * kTiles / 4> b3{};
  constexpr std::integral_constant<int, kTiles> b4{};
  constexpr int kMfmas = kMatrices * TI * TJ;
  constexpr int kDequantOps = kBf16 ? 0 : kTiles * (kPow2 ? 5 : kNvF16 ? 10 : 17);  // vector instructions to dequantize one slice
  constexpr int kLoadsPerTile = kAtoms + (kFp4 || kMxRows ? 1 : 0);
  constexpr int kLoadsPerPhase = (kRowLoads + 3) / 4 + ((kTiles + 3) / 4) * kLoadsPerTile;
  // s_waitcnt vmcnt(kYounger) lgkmcnt(0): everything but the kYounger youngest vector-memory operations is done.
  // Younger than the last A load of step s + 1 (issued during step s - 1, in the last phase that has one) are
  // the weight loads of the later phases of step s - 1 and all loads of phases 1-3 of step s.
  constexpr int kWeightsAfterLastA = a4.value > a3.value ? 0 : a3.value > a2.value ? kTiles - b3.value
                                     : a2.value > a1.value ? kTiles - b2.value : kTiles - b1.value;
  constexpr int kYounger = kWeightsAfterLastA * kLoadsPerTile + a3.value + b3.value * kLoadsPerTile;
  static_assert(kYounger < 64, "vmcnt is a 6-bit counter");
  constexpr int kWaitLanded = (kYounger & 0xF) | (7 << 4) | (0 << 8) | ((kYounger >> 4) << 14);
  constexpr int kWaitAll = (0 & 0xF) | (7 << 4) | (0 << 8) | (0 << 14);  // vmcnt(0) lgkmcnt(0)
  int stage_index = 0;  // s % 3
  // `quarter`: the step's place among four consecutive steps, which is what the block scales' two buffers go by (it is
  // the register set where there are four of them).
  auto iterate = [&](auto set, auto quarter, int step, auto last_steps) __attribute__((always_inline)) {
    constexpr std::integral_constant<int, kFp8A ? set.value % 2 : (quarter.value / 2) % 2> scale_buffer{};
    constexpr std::integral_constant<int, (set.value + 1) % kSets> following{};
    constexpr std::integral_constant<int, (set.value + kSets - 1) % kSets> filling{};
    const int next_index = stage_index == kStages - 1 ? 0 : stage_index + 1;
    const int fill_index = next_index == kStages - 1 ? 0 : next_index + 1;
    u32x4_t* current = lds + stage_index * kStageChunks;
    u32x4_t* next = lds + next_index * kStageChunks;
    u32x4_t* fill = lds + fill_index * kStageChunks;
    const int ahead_a = min(step + 2, steps - 1), ahead_b = min(step + kSets - 1, steps - 1);
    if constexpr (kSplit) {
      // two phases a step: the hi term multiplies while the lo term is read, then the barrier, then the lo term
      // multiplies while the next step's hi term is read; each phase issues half of the step's global loads
      // (With two weight sets the next step's weights are needed at its very start: all of them are issued in the
      // first phase and the A rows in the second, so that the wait for the weights leaves the A rows in flight and
      // neither has less than a phase to land. Issued half and half, the weights were the youngest loads at the
      // step's end and the wait for them drained the memory pipeline every step.)
      constexpr bool kWeightsFirst = kSets == 2;
      constexpr std::integral_constant<int, kWeightsFirst ? 0 : kRowLoads / 2> ah{};
      constexpr std::integral_constant<int, kWeightsFirst ? kTiles : kTiles / 2> bh{};
      constexpr int kSplitMfmas = kMatrices * TI * TJ;
      constexpr int kSplitLoads = ah.value + bh.value * kLoadsPerTile + (kMxRows ? 1 : 0);  // the first phase's, the younger ones at the barrier
      static_assert(kRowLoads % 2 == 0 && kTiles % 2 == 0, "two even halves of loads");
      // younger than the last A load of the step before: only this phase's loads are sure to be
      constexpr int kSplitWait = (kSplitLoads & 0xF) | (7 << 4) | (0 << 8) | ((kSplitLoads >> 4) << 14);
      fetch_term(current, c1);
      multiply_term(set, c0, step, scale_buffer);
      load_a(fill, ahead_a, c0, ah);
      load_a_scales(fill_index, ahead_a);  // (MXFP8 rows: the step's scale dwords, with this phase's loads)
      load_b(filling, ahead_b, c0, bh);
      schedule_phase<0, kSplitMfmas, 2 * TI, 0, 2 * kTiles + 2 * kSplitLoads, kSplitLoads>();
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_waitcnt(last_steps.value ? kWaitAll : kSplitWait);
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
      // block scales: the bytes of the next 128 depths are read from the LDS in the second phase of an even step
      // and formed into words in the second phase of the odd step that follows, one phase before they multiply
      if constexpr (kMxRows) {
        fetch_a_scales(std::integral_constant<int, 1 - set.value % 2>{}, next_index);  // the next step's, landed before the barrier
      } else if constexpr (kFp8Rows) {  // a step is the 128 depths of one scale: the next step's, into the other set
        load_block_scales(min(step + 1, steps - 1));
        form_block_words(std::integral_constant<int, 1 - set.value % 2>{});
      } else {
        if constexpr (kBlockScales && quarter.value % 2 == 0) load_block_scales(min(step / 2 + 1, p.depth / 128 - 1));
        if constexpr (kBlockScales && quarter.value % 2 == 1) form_block_words(std::integral_constant<int, 1 - (quarter.value / 2) % 2>{});
      }
      fetch_term(next, c0);
      multiply_term(set, c1, step, scale_buffer);
      load_a(fill, ahead_a, ah, a4);
      load_b(filling, ahead_b, bh, b4);
      constexpr int kSecondLoads = kRowLoads - ah.value + (kTiles - bh.value) * kLoadsPerTile;
      schedule_phase<0, kSplitMfmas, 2 * TI, 0, 2 * kTiles + 2 * kSecondLoads, kSecondLoads>();
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (kWeightsFirst) {
        // the next step's weights have landed once only this phase's A rows are still in flight (stated here: left
        // to itself the compiler waits for every load before the step's first multiply)
        constexpr int kWeightsLanded = (kSecondLoads & 0xF) | (7 << 4) | (0xF << 8) | ((kSecondLoads >> 4) << 14);
        // The no-op behind the wait is load-bearing. The compiler's own wait insertion treats an LDS-DMA load in flight
        // as a pending access of both memories, so any wait it computes for a register dependency while one is pending is
        // a full drain, vmcnt(0); and where the instruction right behind an explicit s_waitcnt has such a dependency (here
        // the next step's first use of a weight scale), it folds that drain into the explicit wait. With an instruction
        // without operands in between, the explicit count stands, is applied to the compiler's bookkeeping, and the
        // dependency is already met. (Seen in the generated code: vmcnt(0) in every unrolled step but the last, whose wait
        // is followed by the loop's branch. 3.5 % of the split-row paired launch.)
        if (!last_steps.value) {
          __builtin_amdgcn_s_waitcnt(kWeightsLanded);
          asm volatile("s_nop 0");
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      stage_index = next_index;
      return;
    }
    fetch(current, c1, c1);
    dequantize(set, c1, c1, step);
    multiply(c0);
    load_a(fill, ahead_a, c0, a1);
    load_b(filling, ahead_b, c0, b1);
    schedule_phase<0, kMfmas, TI, 0, kDequantOps + 2 * kLoadsPerPhase, kLoadsPerPhase>();
    __builtin_amdgcn_sched_barrier(0);

    fetch(current, c2, c0);
    dequantize(set, c2, c0, step);
    multiply(c1);
    load_a(fill, ahead_a, a1, a2);
    load_b(filling, ahead_b, b1, b2);
    schedule_phase<0, kMfmas, TI, 0, kDequantOps + 2 * kLoadsPerPhase, kLoadsPerPhase>();
    __builtin_amdgcn_sched_barrier(0);

    fetch(current, c3, c1);
    dequantize(set, c3, c1, step);
    multiply(c0);
    load_a(fill, ahead_a, a2, a3);
    load_b(filling, ahead_b, b2, b3);
    schedule_phase<0, kMfmas, TI, 0, kDequantOps + 2 * kLoadsPerPhase, kLoadsPerPhase>();
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    // In the steps after the unrolled loop the compiler drops weight loads nobody consumes, so the count of
    // younger operations no longer holds there: wait for everything (nothing useful is in flight by then).
    __builtin_amdgcn_s_waitcnt(last_steps.value ? kWaitAll : kWaitLanded);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    fetch(next, c0, c0);
    dequantize(following, c0, c0, step + 1);
    multiply(c1);
    load_a(fill, ahead_a, a3, a4);
    load_b(filling, ahead_b, b3, b4);
    schedule_phase<0, kMfmas, TI, 0, kDequantOps + 2 * kLoadsPerPhase, kLoadsPerPhase>();
    __builtin_amdgcn_sched_barrier(0);
    stage_index = next_index;
  };
  load_a(lds, 0, c0, a4);
  load_a(lds + kStageChunks, min(1, steps - 1), c0, a4);
  load_a_scales(0, 0);
  load_a_scales(1, min(1, steps - 1));
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(kWaitAll);
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if constexpr (kFp4) {  // (the same for every lane: kept in scalar registers through the loop)
    tensor_scale0 = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, tensor_scale0)));
    tensor_scale1 = __builtin_bit_cast(float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, tensor_scale1)));
  }
  if constexpr (kSplit) {
    load_block_scales(0);
    form_block_words(c0);
    fetch_a_scales(c0, 0);
    fetch_term(lds, c0);
  } else {
    fetch(lds, c0, c0);
    dequantize(c0, c0, c0, 0);
  }
  int step = 0;
  // Where several blocks share a CU, a wavefront in its main loop goes ahead of one in its set-up or epilogue when both
  // have an instruction to issue, so the matrix pipe is not kept waiting behind address arithmetic and stores (measured:
  // 1 % on the 128-row split tiles' launch, 4 % on a launch of under two tiles a CU; nothing on one block a CU).
  constexpr bool kRaisePriority = BM < 256;
  if constexpr (kRaisePriority) __builtin_amdgcn_s_setprio(3);
  // unrolled so that the register sets, and the block scales' buffers (which turn every four steps), are constants
  constexpr int kUnroll = (kBlockScales && !kFp8A && kSets < 4) ? 4 : kSets;
  static_assert(kUnroll % kSets == 0, "whole rounds of the register sets");
  for (; step + kUnroll <= steps; step += kUnroll) {
    static_range<0>(std::make_integer_sequence<int, kUnroll>{}, [&](auto at) {
      iterate(std::integral_constant<int, decltype(at)::value % kSets>{}, at, step + decltype(at)::value, std::false_type{});
    });
  }
  static_range<0>(std::make_integer_sequence<int, kUnroll - 1>{}, [&](auto at) {  // the last steps % kUnroll steps
    if (step < steps) iterate(std::integral_constant<int, decltype(at)::value % kSets>{}, at, step++, std::true_type{});
  });
  __builtin_amdgcn_s_waitcnt(kWaitAll);  // the clamped tail loads still target the LDS
  if constexpr (kRaisePriority) __builtin_amdgcn_s_setprio(0);

  // ---- epilogue: acc[..][q] is row 8 (q / 4) + 4 (lane / 32) + q % 4, column lane % 32 of its 32 x 32 tile.
  // Neighbouring lanes hold neighbouring columns: each pair of lanes swaps one value so that the even lane
  // holds both columns of row q and the odd lane both of row q + 1. The packed pairs are staged in the LDS the
  // A ring no longer needs, row-major, and the block then writes whole output rows, 16 bytes a lane, so that
  // the tile leaves as full cache lines (direct 4-byte stores of 64-byte row pieces took a quarter of the
  // kernel's time). Tiles of 256 columns are staged in two passes of BM / 2 rows.
  // the 2^8 the decode owes times the expert's tensor scale (src/dew/nn/kernels/gemm.py:660-662)
  // (the scaled instruction applies the block scales themselves, not their 2^-8)
  // (f16 rows: the codes times their block scales as they are, no 2^-8; each row's own 2^s joins below)
  const float factor0 = kFp4 ? (kSplit || kNvF16 ? 1.0f : 256.0f) * tensor_scale0 : 1.0f;
  const float factor1 = kFp4 && PAIRED ? (kSplit || kNvF16 ? 1.0f : 256.0f) * tensor_scale1 : 1.0f;
  float window_factor = 1.0f;
  if constexpr (kWindow) window_factor = (p.factor0 ? *p.factor0 : 1.0f) * (p.factor1 ? *p.factor1 : 1.0f);
  if constexpr (MODE == kPlainF32) {
    // the fp32 sums as they are: a lane group's 32 lanes write 128 contiguous bytes of a row
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int row = wm0 + 32 * i + 8 * (q / 4) + 4 * (lane / 32) + q % 4;
        if (row < valid_rows) {
          float* out_row = p.out_f32 + static_cast<size_t>(row0 + row) * p.width + n0 + wn0 + lane % 32;
#pragma unroll
          for (int j = 0; j < TJ; ++j) out_row[32 * j] = acc[0][i][j][q] * window_factor;
        }
      }
    return;
  }
  constexpr int kPasses = (BN == 256 && BM > 32) ? 2 : 1;
  constexpr int kPassTiles = BM / 32 / kPasses, kPassRows = BM / kPasses;  // row tiles of the block a pass stages
  constexpr int kRowDwords = kOutBN / 2 + 4;  // a staged row: the tile's output columns in bf16 and 16 bytes of padding
  constexpr int kRowChunks = kOutBN / 8;      // 16-byte pieces of an output row
  constexpr int kStoreIters = kPassRows * kRowChunks / kThreads;
  static_assert(kPassRows * kRowChunks % kThreads == 0, "whole store rounds");
  static_assert((BM / 32) % kPasses == 0 && kPassRows * kRowDwords * 4 + BM * 4 <= shared_bytes<BM, BN, MODE>(), "staged tile fits the LDS");
  static_assert(BM <= kThreads, "one thread fetches one row's destination");
  uint32_t* staged = reinterpret_cast<uint32_t*>(lds);
  int* out_row_of = reinterpret_cast<int*>(staged + kPassRows * kRowDwords);  // where each of the tile's rows goes, behind the staged tile
  const bool odd_lane = lane & 1;
  const int out_width = kGated ? p.width / 2 : p.width, out_n0 = kGated ? n0 / 2 : n0;
  // Each expert's bias meets its rows' fp32 sums before their one rounding (src/dew/nn/moe.py:729-742).
  float bias[TJ];
#pragma unroll
  for (int j = 0; j < TJ; ++j)
    bias[j] = (!PAIRED && p.bias) ? p.bias[static_cast<size_t>(expert) * p.width + (kRagged ? min(n0 + wn0 + 32 * j + lane % 32, p.width - 1)
                                                                                               : n0 + wn0 + 32 * j + lane % 32)]
                                  : 0.0f;
  if (p.round_bias) {  // (a caller passes the parameter as it holds it)
#pragma unroll
    for (int j = 0; j < TJ; ++j) bias[j] = bf16_round(bias[j]);
  }
  // quantized rows: a weight block scale that is no normal power of two cannot enter the instruction; the tile is
  // then written as NaN (through the addend every sum meets) rather than as the product under another scale
  if (kFp8Rows && unscalable != 0) {
#pragma unroll
    for (int j = 0; j < TJ; ++j) bias[j] = __uint_as_float(0x7FC00000u);
  }
  // bytes of (neighbour's pair, own pair) that make the lane's staged pair: see the swap below
  const uint32_t swap_select = odd_lane ? 0x03020706u : 0x05040100u;
  const bool plain_swiglu = p.limit <= 0.0f && p.gating == DEW_MOE_GATE_SILU;  // (kernel arguments: the same for the whole launch)
  __builtin_amdgcn_s_barrier();  // every wavefront has read its last A fragments: the ring is free
  if constexpr (!PAIRED) {
    // (the bias has landed: stated here, so that the arithmetic below waits for no load, and the scatter indices, which
    // are fetched next, stay in flight under it)
#pragma unroll
    for (int j = 0; j < TJ; ++j) asm volatile("" : "+v"(bias[j]));
  }
  // Where the tile's rows go: thread t fetches row t's scatter index now, ahead of the arithmetic, and leaves it in a table in
  // the LDS behind the first pass's arithmetic; the store rounds read their rows' entries from there. (Fetched by every
  // thread for each of its store rounds they were up to 16 loads a thread, held in registers through the arithmetic, and
  // where registers were short the compiler moved them aside at once, which waited for them before the arithmetic.)
  int out_row = 0;
  if (tid < BM) {
    const int sorted = row0 + min(tid, valid_rows - 1);
    out_row = p.scatter ? p.scatter[sorted] : sorted;
  }
#pragma unroll
  for (int pass = 0; pass < kPasses; ++pass) {
    if (pass > 0) __syncthreads();  // the previous pass has left the LDS
    // The tile's rounded outputs into the LDS. `plain` (SwiGLU, no clamp) is the same for the whole launch; the choice is made
    // once, around the whole nest, and each side holds cross-lane moves and LDS stores: written as a condition around the
    // arithmetic alone, the compiler evaluated both gates for every output and selected (two exponentials and reciprocals
    // an output; the arithmetic of a 32-row tile's outputs took 6 300 cycles, a tenth of a decode tile's life).
    auto stage_tiles = [&](auto plain) __attribute__((always_inline)) {
#pragma unroll
      for (int i = 0; i < TI; ++i) {
        const int block_tile = wm0 / 32 + i;  // this wavefront's row tile i among the block's
        if (block_tile / kPassTiles != pass) continue;
        const int ii = block_tile % kPassTiles;
        // f16 rows: the 2^s of the lane's 16 rows of this row tile, read ahead of the tile's arithmetic (read where they
        // are used, each read stood behind the staging stores before it and was waited for on its own)
        float row_scale[kNvF16 ? 16 : 1];
        if constexpr (kNvF16) {
#pragma unroll
          for (int q = 0; q < 16; ++q) row_scale[q] = row_factor[wm0 + 32 * i + 8 * (q / 4) + 4 * (lane / 32) + q % 4];
        }
#pragma unroll
        for (int q = 0; q < 16; q += 2) {
          const int row = 32 * ii + 8 * (q / 4) + 4 * (lane / 32) + q % 4 + (odd_lane ? 1 : 0);  // within the pass
#pragma unroll
          for (int j = 0; j < TJ; ++j) {
            if constexpr (kGated) {
              // The even lane holds a gate column and the odd lane the up column beside it, rows q and q + 1 each:
              // the even lane takes the pair of row q, the odd lane the pair of row q + 1, and each writes one value.
              float mine[2];
#pragma unroll
              for (int r = 0; r < 2; ++r) mine[r] = bf16_round(acc[0][i][j][q + r] * factor0 + bias[j]);
              const float sent = odd_lane ? mine[0] : mine[1];
              const float got = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(uint32_t, sent), 0xB1, 0xF, 0xF, true));
              const bf16_t value = odd_lane ? gated_pair_rounded(got, mine[1], p.limit) : gated_pair_rounded(mine[0], got, p.limit);
              reinterpret_cast<bf16_t*>(staged)[row * (2 * kRowDwords) + (wn0 + 32 * j + lane % 32) / 2] = value;
            } else {
              // the lane's rows q (low half) and q + 1 (high half) of its column, rounded
              uint32_t mine;
              if constexpr (PAIRED) {
                // (f16 rows: a row's sums times its own 2^s as well, an exact factor of the expert's)
                const float first0 = kNvF16 ? factor0 * row_scale[kNvF16 ? q : 0] : factor0, first1 = kNvF16 ? factor1 * row_scale[kNvF16 ? q : 0] : factor1;
                const float second0 = kNvF16 ? factor0 * row_scale[kNvF16 ? q + 1 : 0] : factor0, second1 = kNvF16 ? factor1 * row_scale[kNvF16 ? q + 1 : 0] : factor1;
                if constexpr (decltype(plain)::value) {
                  mine = swiglu_rounded(acc[0][i][j][q] * first0, acc[kMatrices - 1][i][j][q] * first1) |
                         (static_cast<uint32_t>(swiglu_rounded(acc[0][i][j][q + 1] * second0, acc[kMatrices - 1][i][j][q + 1] * second1)) << 16);
                } else {  // a clamp or the GeGLU gate
                  mine = gated_rounded(acc[0][i][j][q] * first0, acc[kMatrices - 1][i][j][q] * first1, p.limit, p.gating) |
                         (static_cast<uint32_t>(gated_rounded(acc[0][i][j][q + 1] * second0, acc[kMatrices - 1][i][j][q + 1] * second1, p.limit, p.gating)) << 16);
                }
              } else if constexpr (kFp4) {
                mine = pack_bf16(acc[0][i][j][q] * factor0 + bias[j], acc[0][i][j][q + 1] * factor0 + bias[j]);
              } else if constexpr (kWindow) {
                mine = pack_bf16(acc[0][i][j][q] * window_factor, acc[0][i][j][q + 1] * window_factor);
              } else {
                mine = pack_bf16(acc[0][i][j][q] + bias[j], acc[0][i][j][q + 1] + bias[j]);
              }
              // the even lane keeps row q of both columns and the odd lane row q + 1: each takes the neighbour's pair
              // (quad_perm [1,0,3,2]) and picks its four bytes out of the two pairs with one byte permute
              const uint32_t other = __builtin_amdgcn_mov_dpp(mine, 0xB1, 0xF, 0xF, true);
              const uint32_t packed = __builtin_amdgcn_perm(other, mine, swap_select);
              staged[row * kRowDwords + (wn0 + 32 * j + (lane % 32 & ~1)) / 2] = packed;
            }
          }
        }
      }
    };
    if constexpr (PAIRED) {
      if (plain_swiglu)
        stage_tiles(std::true_type{});
      else
        stage_tiles(std::false_type{});
    } else {
      stage_tiles(std::true_type{});
    }
    if (pass == 0 && tid < BM) out_row_of[tid] = out_row;
    __syncthreads();
    // The thread's pieces of the staged rows and their rows' destinations are all read first, so that no store's address
    // hangs on a load from global memory: each store below stands under its own condition, and with the scatter indices
    // fetched by the storing thread the compiler put a full wait in front of each address, which on this chip waits for the
    // stores before it as well: a pass's eight stores went out one write round trip after another (14 000 cycles of a
    // 128 x 256 tile's 91 000).
    u32x4_t staged_words[kStoreIters];
    int out_rows[kStoreIters];
#pragma unroll
    for (int it = 0; it < kStoreIters; ++it) {
      const int item = tid + it * kThreads;
      staged_words[it] = *reinterpret_cast<const u32x4_t*>(staged + (item / kRowChunks) * kRowDwords + (item % kRowChunks) * 4);
      out_rows[it] = out_row_of[pass * kPassRows + item / kRowChunks];
    }
#pragma unroll
    for (int it = 0; it < kStoreIters; ++it) {
      const int item = tid + it * kThreads;
      const int staged_row = item / kRowChunks, chunk = item % kRowChunks;
      const bool valid = pass * kPassRows + staged_row < valid_rows;
      const u32x4_t words = staged_words[it];
      if constexpr (kSplitOut) {
        // The row's 128 columns of this tile as two e4m3 terms under one scale (dew_moe_split_rows' arithmetic on a
        // 128-column block): the 16 lanes that hold the row's chunks agree on its largest exponent field, each
        // converts its 8 values and writes their hi and lo bytes where the scaled instruction's operand order puts
        // them (split.hip: each 64 depths as [group 0 hi][group 0 lo][group 1 hi][group 1 lo]).
        static_assert(!kSplitOut || kRowChunks == 16, "a row's chunks fill one 16-lane row of the wavefront");
        uint32_t largest = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) largest = max(largest, max((words[i] >> 7) & 0xFFu, (words[i] >> 23) & 0xFFu));
        largest = max(largest, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(largest), 0xB1, 0xF, 0xF, true)));   // lane ^ 1
        largest = max(largest, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(largest), 0x4E, 0xF, 0xF, true)));   // lane ^ 2
        largest = max(largest, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(largest), 0x141, 0xF, 0xF, true)));  // 7 - lane in each 8
        largest = max(largest, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(largest), 0x140, 0xF, 0xF, true)));  // 15 - lane
        const int field = min(max(static_cast<int>(largest), 16), 254);
        const int hi_byte = field - 7;
        const float inverse = __uint_as_float(static_cast<uint32_t>(254 - hi_byte) << 23);
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[2 * i] = __uint_as_float(words[i] << 16) * inverse;
          v[2 * i + 1] = __uint_as_float(words[i] & 0xFFFF0000u) * inverse;
        }
        uint32_t hi[2], lo[2];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          hi[w] = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w], v[4 * w + 1], 0, false);
          hi[w] = __builtin_amdgcn_cvt_pk_fp8_f32(v[4 * w + 2], v[4 * w + 3], hi[w], true);
          const auto first = __builtin_amdgcn_cvt_pk_f32_fp8(hi[w], false), second = __builtin_amdgcn_cvt_pk_f32_fp8(hi[w], true);
          lo[w] = __builtin_amdgcn_cvt_pk_fp8_f32((v[4 * w] - first[0]) * 16.0f, (v[4 * w + 1] - first[1]) * 16.0f, 0, false);
          lo[w] = __builtin_amdgcn_cvt_pk_fp8_f32((v[4 * w + 2] - second[0]) * 16.0f, (v[4 * w + 3] - second[1]) * 16.0f, lo[w], true);
        }
        if (valid) {
          const int within = chunk % 8, half = within / 4, group = (within % 4) / 2, piece = within % 2;
          uint8_t* block = reinterpret_cast<uint8_t*>(p.out + static_cast<size_t>(out_rows[it]) * out_width + out_n0) +
                           (chunk / 8) * 128 + group * 64 + half * 16 + piece * 8;
          *reinterpret_cast<uint32_t*>(block) = hi[0];
          *reinterpret_cast<uint32_t*>(block + 4) = hi[1];
          *reinterpret_cast<uint32_t*>(block + 32) = lo[0];
          *reinterpret_cast<uint32_t*>(block + 36) = lo[1];
          if (chunk == 0)
            p.out_scale[static_cast<size_t>(row0 + pass * kPassRows + staged_row) * block_scale_pitch(p.width) + n0 / 128] = static_cast<uint8_t>(hi_byte);
        }
      } else {
        if (valid && (!kRagged || out_n0 + chunk * 8 < out_width))
          *reinterpret_cast<u32x4_t*>(p.out + static_cast<size_t>(out_rows[it]) * out_width + out_n0 + chunk * 8) = words;
      }
    }
  }
}

static int check_bank(const char* who, const dew_moe_bank* bank, const char* name) {
  DEW_REQUIRE(bank, "%s: %s bank must not be null", who, name);
  DEW_REQUIRE(bank->layout == DEW_MOE_LAYOUT_PREPARED, "%s: %s bank is in the reference layout; call dew_moe_prepare_bank once at load", who, name);
  DEW_REQUIRE(bank->format == DEW_MOE_W_FP8_BLOCK || bank->format == DEW_MOE_W_FP8_CHANNEL || bank->format == DEW_MOE_W_NVFP4 ||
                  bank->format == DEW_MOE_W_MXFP4 || bank->format == DEW_MOE_W_MXFP8 || bank->format == DEW_MOE_W_BF16,
              "%s: %s bank has unknown format %d", who, name, bank->format);
  DEW_REQUIRE(bank->experts >= 1 && bank->experts <= 4096, "%s: %s bank has %d experts", who, name, bank->experts);
  if (bank->format == DEW_MOE_W_BF16 || bank->format == DEW_MOE_W_MXFP4 || bank->format == DEW_MOE_W_NVFP4) {  // whole 64-deep steps and 32-column atoms
    DEW_REQUIRE(bank->depth >= 128 && bank->depth % 64 == 0, "%s: %s bank depth %d is not a multiple of 64", who, name, bank->depth);
    DEW_REQUIRE(bank->width >= 128 && bank->width % 32 == 0, "%s: %s bank width %d is not a multiple of 32", who, name, bank->width);
  } else {
    DEW_REQUIRE(bank->depth >= 128 && bank->depth % 128 == 0, "%s: %s bank depth %d is not a multiple of 128", who, name, bank->depth);
    DEW_REQUIRE(bank->width % 128 == 0 && bank->width >= 128, "%s: %s bank width %d is not a multiple of 128", who, name, bank->width);
  }
  DEW_REQUIRE(bank->depth <= 128 * kMaxDepthBlocks, "%s: %s bank depth %d is above %d", who, name, bank->depth, 128 * kMaxDepthBlocks);
  DEW_REQUIRE(bank->codes && (bank->scales || bank->format == DEW_MOE_W_BF16), "%s: %s bank codes and scales must not be null", who, name);
  DEW_REQUIRE((bank->format != DEW_MOE_W_NVFP4 && bank->format != DEW_MOE_W_MXFP4) || bank->tensor_scale, "%s: %s NVFP4 bank needs tensor scales", who, name);
  DEW_REQUIRE(aligned16(bank->codes), "%s: %s bank codes must be 16-byte aligned", who, name);
  return DEW_MOE_OK;
}

// The split-row launches read their rows' scales and their weights in whole 128-deep blocks and write whole 128-column strips.
static int check_split_extents(const char* who, const dew_moe_bank* bank, const char* name) {
  DEW_REQUIRE(bank->depth % 128 == 0 && bank->width % 128 == 0, "%s: %s bank [%d, %d] on split rows: depth and width are whole 128s", who, name,
              bank->depth, bank->width);
  return DEW_MOE_OK;
}

template <int FORMAT, int MODE, int BM, int BN, int WM, int WN>
static int launch_tile(const char* who, GemmParams p, hipStream_t stream) {
  // block-scaled activations keep their tile's scales behind the ring (reserved at their largest: kMaxBlockScaleDepth)
  constexpr size_t kShared = shared_bytes<BM, BN, MODE>() +
                             (FORMAT == kFormatMxSplitBlocks || FORMAT == kFormatFp8Rows ? static_cast<size_t>(BM) * block_scale_pitch(kMaxBlockScaleDepth) : 0) +
                             (FORMAT == kFormatMxFp8Rows || FORMAT == kFormatMxFp8Window ? 3 * static_cast<size_t>(BM) * 4 : 0);  // MXFP8 rows: a dword a row a stage
  auto kernel = grouped_gemm_kernel<FORMAT, MODE, BM, BN, WM, WN>;
  static std::once_flag configured;  // dynamic LDS above 64 KiB must be opted into once per kernel (whichever thread calls first)
  static hipError_t reserved = hipSuccess;
  std::call_once(configured, [&] {
    reserved = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kShared));
  });
  if (reserved != hipSuccess) return fail(DEW_MOE_ELAUNCH, "%s: cannot reserve %zu bytes of LDS", who, kShared);
  // every expert may end in a partial tile, and the zeroed tail may add one more
  p.m_tile_bound = p.tail_of > 0 ? p.experts : (p.rows + BM - 1) / BM + p.experts + 1;
  if (FORMAT == kFormatMxFp8Window || FORMAT == kFormatBf16Window) p.m_tile_bound = p.experts * ((p.window_rows + BM - 1) / BM);  // every group the same whole rows
  const int total = p.m_tile_bound * ((p.width + BN - 1) / BN);
  // A chunk is 4 m-tiles x 8 strips, and 2 x 8 for the 256-row tiles, whose launches have the fewest tiles: dealt in
  // smaller chunks their last round spreads more evenly over the XCDs (measured on 16 to 64 m-tiles of 256 rows: the down
  // launch 8 % shorter, the paired one 3 %; taller chunks of 8 or 16 m-tiles, which fetch less, were slower everywhere)
  p.group_m = BM == 256 ? 2 : 4;
  // (a one-bank launch of few tiles likewise: C5's down launch, 1 168 tiles of 128 rows, runs its step 1 % shorter dealt in
  // chunks of 16; the paired launches are best at 4 x 8 down to the decode sizes)
  if (MODE != kSwigluOfTwo && MODE != kSwigluOfTwoSplit && total < 2048) p.group_m = 2;
  const int round = 64 * p.group_m;
  const int blocks = ((total + round - 1) / round) * round;  // whole chunks of tiles for each of the 8 XCDs
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(kThreads), kShared, stream, p);
  return launched(who);
}

// Rows of the block tile, from what the host knows (rows and experts; the routing itself stays on the device).
// Three rules, measured over ragged groups (sizes spread an eighth around their mean) of 8 .. 2048 rows on four model
// shapes. Fill: a group's last tile is half empty on average, so the tile is about as tall as the average group while
// what the shorter tile loses when full (it reads and converts the weights again for half the rows: 15 to 26 % on an
// FP8 bank, 5 to 11 % on one whose codes cost the vector unit little) is less than what the taller one multiplies
// of empty rows: 32-row tiles up to 26 rows a group (at 32, half the groups need a second, nearly empty one and
// 64-row tiles are 15 to 25 % faster), 64-row tiles up to 72 rows on FP8 banks (and from 129 to 184, where three
// of them cover what two 128-row tiles would, 5 to 10 % faster) and up to 384 on the cheap ones.
// Occupancy: a launch of fewer tiles than CUs halves its tile until there are enough (8 experts x 512 rows x 512
// columns: 144 tiles of 128 rows take 16.5 us, 272 tiles of 64 rows 11.7 us). 256-row tiles, which fill every
// accumulator register, are kept to the cheap banks and to groups of 2048 rows or more. Decode-sized groups take the
// 32-row tile, whose four wavefronts split the columns, so that thousands of wavefronts stream the weights at once.
static thread_local int forced_tile_rows = 0;  // dew_moe_tile_rows, per calling thread: 0 leaves the choice to the rules below

static int tile_rows(const GemmParams& p, bool cheap) {
  if (forced_tile_rows != 0) return forced_tile_rows;
  const int average = p.rows / p.experts;
  if (cheap && average >= 2048 && p.width % 256 == 0) return 256;  // below, two 128-row blocks a CU are 2 to 5 % faster
  int rows = average <= 26 ? 32 : average <= (cheap ? 384 : 72) || (average > 128 && average <= 184) ? 64 : 128;
  const long long strips = p.width / 128;
  // (of 128-row tiles a launch wants one and a half a CU: at 288 and 376 of them, 8 experts x 512 and 700 rows x 1024
  // columns, 64-row tiles are 5 to 13 % faster on FP8 and NVFP4 banks; at 432 and 448, on deeper banks, 17 % slower)
  while (rows > 32 && (p.rows / rows + p.experts / 2) * strips < (rows == 128 ? 400 : 256)) rows /= 2;
  return rows;
}

template <int FORMAT, int MODE>
static int launch_format(const char* who, const GemmParams& p, hipStream_t stream) {
  // (256-row tiles: the banks whose weights cost the vector unit little or nothing to bring to bf16. General NVFP4
  // scales cost it as much as FP8 does: two 128-row blocks a CU run a paired launch of 1024-row groups 7 to 15 % faster
  // than one 256-row block; a one-bank launch the same there and 4 to 7 % slower on 4096-row groups, so it keeps the taller tile)
  constexpr bool kPaired = MODE == kSwigluOfTwo;
  constexpr bool kFp4 = FORMAT == DEW_MOE_W_MXFP4 || FORMAT == DEW_MOE_W_BF16 || (FORMAT == DEW_MOE_W_NVFP4 && !kPaired);
  switch (tile_rows(p, kFp4)) {
    case 32:
      // one bank: 256 columns a block where that still leaves every CU several blocks, so that a launch is one round
      if (!kPaired && p.width % 256 == 0 && static_cast<long long>(p.experts) * (p.width / 256) >= 768)
        return launch_tile<FORMAT, MODE, 32, 256, 1, 4>(who, p, stream);
      // (an FP4 bank's step brings half an FP8 one's bytes for the same rows' worth of LDS traffic and barriers, so the wider
      // block pays sooner, and its widths need not be whole 256s: 32 experts x 5760 columns, 736 blocks, 59 -> 54 us; at 384
      // blocks, 32 x 2880, it is 7 % slower than 128 columns)
      if (!kPaired && (FORMAT == DEW_MOE_W_MXFP4 || FORMAT == DEW_MOE_W_NVFP4) && static_cast<long long>(p.experts) * ((p.width + 255) / 256) >= 640)
        return launch_tile<FORMAT, MODE, 32, 256, 1, 4>(who, p, stream);
      return launch_tile<FORMAT, MODE, 32, 128, 1, 4>(who, p, stream);
    case 64:
      return launch_tile<FORMAT, MODE, 64, 128, 1, 4>(who, p, stream);
    case 256:
      if (kPaired || p.width % 256 == 0) return launch_tile<FORMAT, MODE, 256, kPaired ? 128 : 256, 1, 4>(who, p, stream);
      [[fallthrough]];  // one bank whose width is not whole 256s: the 128-row tile
    default: {
      // Last tiles of at most 64 rows can go to a second launch of 64-row tiles. That launch runs after the first, so
      // it pays only where it fills the chip by itself and most groups have such a last tile: the average group just
      // over a whole number of tiles (256 groups of 256 +- 16 rows: 2.5 tiles a group become 2 and a 64-row one, 1.5
      // to 2.5 % faster; at 160 or 200 rows a group the same two launches are 5 to 15 % slower than one, a bank of 8
      // experts, whose few last tiles run their whole depth alone, 20 to 35 % slower, and groups of 1024 rows 1 %).
      const int average = p.rows / p.experts;
      const bool shared = forced_tile_rows == 0 && average >= 128 && average < 512 && average % 128 <= 40 &&
                          static_cast<long long>(p.experts) * (p.width / 128) >= 512;
      GemmParams taller = p;
      taller.skip_tails = shared ? 64 : 0;
      int status;
      if (!kPaired && p.width % 256 == 0 && static_cast<long long>(p.rows / 128 + 1) * (p.width / 256) >= 512)
        status = launch_tile<FORMAT, MODE, 128, 256, 1, 4>(who, taller, stream);  // enough tiles to fill the chip twice over
      else
        status = launch_tile<FORMAT, MODE, 128, 128, 1, 4>(who, taller, stream);
      if (status != DEW_MOE_OK || !shared) return status;
      GemmParams rest = p;
      rest.tail_of = 128;
      return launch_tile<FORMAT, MODE, 64, 128, 1, 4>(who, rest, stream);
    }
  }
}

template <int MODE>
static int launch(const char* who, const GemmParams& p, int format, hipStream_t stream) {
  switch (format) {
    case DEW_MOE_W_FP8_BLOCK:
      return launch_format<DEW_MOE_W_FP8_BLOCK, MODE>(who, p, stream);
    case DEW_MOE_W_FP8_CHANNEL:
      return launch_format<DEW_MOE_W_FP8_CHANNEL, MODE>(who, p, stream);
    case DEW_MOE_W_MXFP4:
      return launch_format<DEW_MOE_W_MXFP4, MODE>(who, p, stream);
    case DEW_MOE_W_BF16:
      return launch_format<DEW_MOE_W_BF16, MODE>(who, p, stream);
    case DEW_MOE_W_MXFP8:
      return fail(DEW_MOE_EINVAL, "%s: an MXFP8 bank multiplies MXFP8 rows (dew_moe_grouped_gemm_mxfp8_rows), not bf16 rows", who);
    default:
      return launch_format<DEW_MOE_W_NVFP4, MODE>(who, p, stream);
  }
}

static int fill_single(const char* who, GemmParams& p, const void* x, const int32_t* gather, const int32_t* offsets,
                       const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out, int32_t rows,
                       const int32_t* sizes = nullptr) {
  DEW_REQUIRE(x && (offsets || sizes) && out, "%s: x, the groups' offsets (or sizes) and out must not be null", who);
  p.sizes = sizes;
  DEW_REQUIRE(aligned16(x) && aligned16(out), "%s: x and out must be 16-byte aligned", who);
  p.x = static_cast<const bf16_t*>(x);
  p.gather = gather;
  p.offsets = offsets;
  p.scatter = scatter;
  p.w0 = BankView{static_cast<const uint8_t*>(w->codes), w->scales, w->tensor_scale};
  p.w1 = p.w0;
  p.out = static_cast<bf16_t*>(out);
  p.bias = bias;
  p.experts = w->experts;
  p.depth = w->depth;
  p.width = w->width;
  p.rows = rows;
  return DEW_MOE_OK;
}

}  // namespace dew

extern "C" int dew_moe_tile_rows(int32_t rows) {
  using namespace dew;
  DEW_REQUIRE(rows == 0 || rows == 32 || rows == 64 || rows == 128 || rows == 256,
              "dew_moe_tile_rows: tiles are 32, 64, 128 or 256 rows (0 = chosen per launch), not %d", rows);
  forced_tile_rows = rows;
  return DEW_MOE_OK;
}

static int grouped_gemm_of(const char* who, const void* x, const int32_t* gather, const int32_t* offsets, const int32_t* sizes,
                           const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out, int32_t rows, void* stream,
                           bool round_bias = false) {
  using namespace dew;
  if (int rc = check_bank(who, w, "weight")) return rc;
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  GemmParams p{};
  if (int rc = fill_single(who, p, x, gather, offsets, w, bias, scatter, out, rows, sizes)) return rc;
  p.round_bias = round_bias ? 1 : 0;
  return launch<kPlain>(who, p, w->format, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_grouped_gemm_bias(const void* x, const int32_t* gather, const int32_t* offsets,
                                         const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out,
                                         int32_t rows, void* stream) {
  return grouped_gemm_of("dew_moe_grouped_gemm", x, gather, offsets, nullptr, w, bias, scatter, out, rows, stream);
}

extern "C" int dew_moe_grouped_gemm_param_bias(const void* x, const int32_t* gather, const int32_t* offsets, const int32_t* group_sizes,
                                               const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out,
                                               int32_t rows, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows == 0 || (offsets != nullptr) != (group_sizes != nullptr),
              "dew_moe_grouped_gemm_param_bias: the groups come as offsets [E + 1] or as group_sizes [E], one of them");
  return grouped_gemm_of("dew_moe_grouped_gemm_param_bias", x, gather, offsets, group_sizes, w, bias, scatter, out, rows, stream, true);
}

extern "C" int dew_moe_grouped_gemm_sizes(const void* x, const int32_t* gather, const int32_t* group_sizes,
                                          const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out,
                                          int32_t rows, void* stream) {
  return grouped_gemm_of("dew_moe_grouped_gemm_sizes", x, gather, nullptr, group_sizes, w, bias, scatter, out, rows, stream);
}

extern "C" int dew_moe_grouped_gemm(const void* x, const int32_t* gather, const int32_t* offsets,
                                    const dew_moe_bank* w, const int32_t* scatter, void* out, int32_t rows,
                                    void* stream) {
  return dew_moe_grouped_gemm_bias(x, gather, offsets, w, nullptr, scatter, out, rows, stream);
}

extern "C" int dew_moe_grouped_gemm_split(const void* x_split, const uint8_t* x_scale, const int32_t* gather, const int32_t* offsets,
                                          const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out,
                                          int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_grouped_gemm_split";
  if (int rc = check_bank(who, w, "weight")) return rc;
  if (int rc = check_split_extents(who, w, "weight")) return rc;
  DEW_REQUIRE(w->format == DEW_MOE_W_MXFP4 && w->width % 256 == 0,
              "%s: split activations multiply an MXFP4 bank (power-of-two block scales) whose width is whole 256s; this one is "
              "format %d, width %d", who, w->format, w->width);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x_scale, "%s: the rows' scales must not be null", who);
  GemmParams p{};
  if (int rc = fill_single(who, p, x_split, gather, offsets, w, bias, scatter, out, rows)) return rc;
  p.a_scale = x_scale;
  return launch_tile<kFormatMxSplit, kPlain, 256, 256, 2, 2>(who, p, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_gateup_swiglu_split(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                                           const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden,
                                           int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_gateup_swiglu_split";
  if (int rc = check_bank(who, gate, "gate")) return rc;
  if (int rc = check_bank(who, up, "up")) return rc;
  if (int rc = check_split_extents(who, gate, "gate")) return rc;
  if (int rc = check_split_extents(who, up, "up")) return rc;
  DEW_REQUIRE(gate->format == DEW_MOE_W_MXFP4 && up->format == DEW_MOE_W_MXFP4,
              "%s: split activations multiply MXFP4 banks (power-of-two block scales); these are formats %d and %d", who,
              gate->format, up->format);
  DEW_REQUIRE(gate->experts == up->experts && gate->depth == up->depth && gate->width == up->width,
              "%s: gate [%d, %d, %d] and up [%d, %d, %d] differ", who, gate->experts, gate->depth, gate->width, up->experts,
              up->depth, up->width);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x_split && x_scale && offsets && hidden, "%s: x_split, x_scale, offsets and hidden must not be null", who);
  DEW_REQUIRE(aligned16(x_split) && aligned16(hidden), "%s: x_split and hidden must be 16-byte aligned", who);
  GemmParams p{};
  p.x = static_cast<const bf16_t*>(x_split);
  p.a_scale = x_scale;
  p.gather = gather;
  p.offsets = offsets;
  p.w0 = BankView{static_cast<const uint8_t*>(gate->codes), gate->scales, gate->tensor_scale};
  p.w1 = BankView{static_cast<const uint8_t*>(up->codes), up->scales, up->tensor_scale};
  p.out = static_cast<bf16_t*>(hidden);
  p.experts = gate->experts;
  p.depth = gate->depth;
  p.width = gate->width;
  p.rows = rows;
  return launch_tile<kFormatMxSplit, kSwigluOfTwo, 256, 128, 2, 2>(who, p, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_grouped_gemm_split_blocks(const void* x_split, const uint8_t* x_scales, const int32_t* gather,
                                                 const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                                                 const int32_t* scatter, void* out, int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_grouped_gemm_split_blocks";
  if (int rc = check_bank(who, w, "weight")) return rc;
  if (int rc = check_split_extents(who, w, "weight")) return rc;
  DEW_REQUIRE(w->format == DEW_MOE_W_MXFP4 && w->width % 256 == 0,
              "%s: split activations multiply an MXFP4 bank (power-of-two block scales) whose width is whole 256s; this one is "
              "format %d, width %d", who, w->format, w->width);
  DEW_REQUIRE(w->depth <= kMaxBlockScaleDepth, "%s: bank depth %d is above %d (a tile's block scales are kept in the LDS)", who,
              w->depth, kMaxBlockScaleDepth);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x_scales && aligned16(x_scales), "%s: the rows' scales must not be null and must be 16-byte aligned", who);
  GemmParams p{};
  if (int rc = fill_single(who, p, x_split, gather, offsets, w, bias, scatter, out, rows)) return rc;
  p.a_scale = x_scales;
  if (forced_tile_rows == 128) return launch_tile<kFormatMxSplitBlocks, kPlain, 128, 256, 2, 2>(who, p, static_cast<hipStream_t>(stream));
  return launch_tile<kFormatMxSplitBlocks, kPlain, 256, 256, 2, 2>(who, p, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_grouped_gemm_fp8_rows(const void* x_codes, const uint8_t* x_scales, const int32_t* gather,
                                             const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                                             const int32_t* scatter, void* out, int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_grouped_gemm_fp8_rows";
  if (int rc = check_bank(who, w, "weight")) return rc;
  DEW_REQUIRE(w->format == DEW_MOE_W_FP8_BLOCK, "%s: quantized rows multiply an FP8 128 x 128 block bank; this one is format %d", who,
              w->format);
  DEW_REQUIRE(w->depth <= kMaxBlockScaleDepth, "%s: bank depth %d is above %d (a tile's block scales are kept in the LDS)", who,
              w->depth, kMaxBlockScaleDepth);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x_scales && aligned16(x_scales), "%s: the rows' scales must not be null and must be 16-byte aligned", who);
  GemmParams p{};
  if (int rc = fill_single(who, p, x_codes, gather, offsets, w, bias, scatter, out, rows)) return rc;
  p.a_scale = x_scales;
  if (p.width % 256 == 0) return launch_tile<kFormatFp8Rows, kPlain, 256, 256, 2, 2>(who, p, static_cast<hipStream_t>(stream));
  return launch_tile<kFormatFp8Rows, kPlain, 256, 128, 2, 2>(who, p, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_grouped_gemm_mxfp8_rows(const void* x_codes, const uint8_t* x_scales, const int32_t* gather,
                                               const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                                               const int32_t* scatter, void* out, int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_grouped_gemm_mxfp8_rows";
  if (int rc = check_bank(who, w, "weight")) return rc;
  DEW_REQUIRE(w->format == DEW_MOE_W_MXFP8, "%s: MXFP8 rows multiply an MXFP8 bank; this one is format %d", who, w->format);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x_scales && (reinterpret_cast<uintptr_t>(x_scales) & 3u) == 0, "%s: the rows' scales must not be null and must be 4-byte aligned", who);
  GemmParams p{};
  if (int rc = fill_single(who, p, x_codes, gather, offsets, w, bias, scatter, out, rows)) return rc;
  p.a_scale = x_scales;
  if (p.width % 256 == 0) return launch_tile<kFormatMxFp8Rows, kPlain, 256, 256, 2, 2>(who, p, static_cast<hipStream_t>(stream));
  return launch_tile<kFormatMxFp8Rows, kPlain, 256, 128, 2, 2>(who, p, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_kernel_gradient_mxfp8(const void* lhs_t_codes, const uint8_t* lhs_t_scales, const dew_moe_bank* rhs_t,
                                             const int32_t* offsets, void* out, int32_t out_is_f32, int32_t depth, int32_t groups,
                                             void* stream) {
  using namespace dew;
  const char* who = "dew_moe_kernel_gradient_mxfp8";
  DEW_REQUIRE(rhs_t, "%s: the rhs_t bank must not be null", who);
  DEW_REQUIRE(rhs_t->format == DEW_MOE_W_MXFP8 && rhs_t->layout == DEW_MOE_LAYOUT_PREPARED && rhs_t->experts == 1,
              "%s: rhs_t is one prepared MXFP8 matrix [width, tokens] (dew_moe_quantize_columns_*, as a bank), not format %d, layout %d, %d experts",
              who, rhs_t->format, rhs_t->layout, rhs_t->experts);
  const int tokens = rhs_t->depth;
  DEW_REQUIRE(tokens >= 0 && tokens % 128 == 0, "%s: %d tokens are not whole 128-token blocks", who, tokens);
  DEW_REQUIRE(rhs_t->width >= 128 && rhs_t->width % 128 == 0, "%s: width %d is not a multiple of 128", who, rhs_t->width);
  DEW_REQUIRE(depth >= 128 && depth % 128 == 0, "%s: depth %d is not a multiple of 128", who, depth);
  DEW_REQUIRE(groups >= 1 && groups <= 4096, "%s: %d groups", who, groups);
  DEW_REQUIRE(static_cast<long long>(groups) * depth < (1ll << 31), "%s: %d groups of %d rows overflow the row index", who, groups, depth);
  DEW_REQUIRE(offsets && out && aligned16(out), "%s: offsets and out must not be null, out 16-byte aligned", who);
  DEW_REQUIRE(tokens == 0 || (lhs_t_codes && lhs_t_scales && rhs_t->codes && rhs_t->scales), "%s: the operands' codes and scales must not be null", who);
  DEW_REQUIRE(aligned16(lhs_t_codes) && aligned16(rhs_t->codes) && (reinterpret_cast<uintptr_t>(lhs_t_scales) & 3u) == 0,
              "%s: codes must be 16-byte and the lhs_t's scales 4-byte aligned", who);
  GemmParams p{};
  p.x = static_cast<const bf16_t*>(lhs_t_codes);
  p.a_scale = lhs_t_scales;
  p.windows = offsets;
  p.window_rows = depth;
  p.w0 = BankView{static_cast<const uint8_t*>(rhs_t->codes), rhs_t->scales, nullptr};
  p.w1 = p.w0;
  p.out = static_cast<bf16_t*>(out);
  p.out_f32 = static_cast<float*>(out);
  p.experts = groups;
  p.depth = tokens;
  p.width = rhs_t->width;
  p.rows = groups * depth;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (out_is_f32) {
    if (p.width % 256 == 0) return launch_tile<kFormatMxFp8Window, kPlainF32, 256, 256, 2, 2>(who, p, s);
    return launch_tile<kFormatMxFp8Window, kPlainF32, 256, 128, 2, 2>(who, p, s);
  }
  if (p.width % 256 == 0) return launch_tile<kFormatMxFp8Window, kPlain, 256, 256, 2, 2>(who, p, s);
  return launch_tile<kFormatMxFp8Window, kPlain, 256, 128, 2, 2>(who, p, s);
}

extern "C" int dew_moe_kernel_gradient_bf16(const void* lhs_t, const dew_moe_bank* rhs_t, const int32_t* offsets, const float* lhs_scale,
                                            const float* rhs_scale, void* out, int32_t out_is_f32, int32_t depth, int32_t groups,
                                            void* stream) {
  using namespace dew;
  const char* who = "dew_moe_kernel_gradient_bf16";
  DEW_REQUIRE(rhs_t, "%s: the rhs_t bank must not be null", who);
  DEW_REQUIRE(rhs_t->format == DEW_MOE_W_BF16 && rhs_t->layout == DEW_MOE_LAYOUT_PREPARED && rhs_t->experts == 1,
              "%s: rhs_t is one prepared bf16 matrix [width, tokens] (dew_moe_transpose_columns, as a bank), not format %d, layout %d, %d experts",
              who, rhs_t->format, rhs_t->layout, rhs_t->experts);
  const int tokens = rhs_t->depth;
  DEW_REQUIRE(tokens >= 0 && tokens % 128 == 0, "%s: %d tokens are not whole 128s", who, tokens);
  DEW_REQUIRE(rhs_t->width >= 128 && rhs_t->width % 128 == 0, "%s: width %d is not a multiple of 128", who, rhs_t->width);
  DEW_REQUIRE(depth >= 128 && depth % 128 == 0, "%s: depth %d is not a multiple of 128", who, depth);
  DEW_REQUIRE(groups >= 1 && groups <= 4096, "%s: %d groups", who, groups);
  DEW_REQUIRE(static_cast<long long>(groups) * depth < (1ll << 31), "%s: %d groups of %d rows overflow the row index", who, groups, depth);
  DEW_REQUIRE(offsets && out && aligned16(out), "%s: offsets and out must not be null, out 16-byte aligned", who);
  DEW_REQUIRE(tokens == 0 || (lhs_t && rhs_t->codes), "%s: the operands must not be null", who);
  DEW_REQUIRE(aligned16(lhs_t) && aligned16(rhs_t->codes), "%s: the operands must be 16-byte aligned", who);
  GemmParams p{};
  p.x = static_cast<const bf16_t*>(lhs_t);
  p.windows = offsets;
  p.window_rows = depth;
  p.factor0 = lhs_scale;
  p.factor1 = rhs_scale;
  p.w0 = BankView{static_cast<const uint8_t*>(rhs_t->codes), nullptr, nullptr};
  p.w1 = p.w0;
  p.out = static_cast<bf16_t*>(out);
  p.out_f32 = static_cast<float*>(out);
  p.experts = groups;
  p.depth = tokens;
  p.width = rhs_t->width;
  p.rows = groups * depth;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (out_is_f32) {
    if (p.width % 256 == 0) return launch_tile<kFormatBf16Window, kPlainF32, 256, 256, 1, 4>(who, p, s);
    return launch_tile<kFormatBf16Window, kPlainF32, 256, 128, 1, 4>(who, p, s);
  }
  if (p.width % 256 == 0) return launch_tile<kFormatBf16Window, kPlain, 256, 256, 1, 4>(who, p, s);
  return launch_tile<kFormatBf16Window, kPlain, 256, 128, 1, 4>(who, p, s);
}

namespace dew {

// The paired launch on split rows whose gated rows leave split as well; `terms`: the rows' terms (DEW_MOE_SECOND_TERM_*).
static int gateup_split_out_of(const char* who, int terms, const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                               const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden_split,
                               uint8_t* hidden_scales, int32_t rows, void* stream, int32_t activation, float limit) {
  if (int rc = check_bank(who, gate, "gate")) return rc;
  if (int rc = check_bank(who, up, "up")) return rc;
  if (int rc = check_split_extents(who, gate, "gate")) return rc;
  if (int rc = check_split_extents(who, up, "up")) return rc;
  DEW_REQUIRE(gate->format == DEW_MOE_W_MXFP4 && up->format == DEW_MOE_W_MXFP4,
              "%s: split activations multiply MXFP4 banks (power-of-two block scales); these are formats %d and %d", who,
              gate->format, up->format);
  DEW_REQUIRE(gate->experts == up->experts && gate->depth == up->depth && gate->width == up->width,
              "%s: gate [%d, %d, %d] and up [%d, %d, %d] differ", who, gate->experts, gate->depth, gate->width, up->experts,
              up->depth, up->width);
  DEW_REQUIRE(activation == DEW_MOE_GATE_SILU || activation == DEW_MOE_GATE_GELU_TANH,
              "%s: the gate's activation %d is neither silu (0: swiglu) nor the tanh gelu (1: geglu)", who, activation);
  DEW_REQUIRE(limit >= 0.0f, "%s: the clamp limit %g must be positive (0: none)", who, static_cast<double>(limit));
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x_split && (x_scale || terms == DEW_MOE_TERMS_E2M3_PAIR) && offsets && hidden_split && hidden_scales,
              "%s: x_split, x_scale, offsets, hidden_split and hidden_scales must not be null", who);
  DEW_REQUIRE(aligned16(x_split) && aligned16(hidden_split), "%s: x_split and hidden_split must be 16-byte aligned", who);
  GemmParams p{};
  p.x = static_cast<const bf16_t*>(x_split);
  p.a_scale = x_scale;
  p.gather = gather;
  p.offsets = offsets;
  p.w0 = BankView{static_cast<const uint8_t*>(gate->codes), gate->scales, gate->tensor_scale};
  p.w1 = BankView{static_cast<const uint8_t*>(up->codes), up->scales, up->tensor_scale};
  p.out = static_cast<bf16_t*>(hidden_split);
  p.out_scale = hidden_scales;
  p.experts = gate->experts;
  p.depth = gate->depth;
  p.width = gate->width;
  p.rows = rows;
  p.gating = activation;
  p.limit = limit > 0.0f ? bf16_round_host(limit) : 0.0f;
  // 128-row tiles at two blocks a CU (256 registers a lane, two weight register sets): one block's tile search, first
  // loads and epilogue run under the other's main loop. Measured on 8 experts x 4096 rows of 4096 x 14336: 5.18 ms
  // against 5.30 ms for 256-row tiles at one block a CU, the same bits. (The plain product stays on 256-row
  // tiles: 2.55 against 2.61 ms.)
  const hipStream_t s = static_cast<hipStream_t>(stream);
  if (terms == DEW_MOE_TERMS_E2M3_PAIR) {
    if (forced_tile_rows == 256) return launch_tile<kFormatMxSplit66, kSwigluOfTwoSplit, 256, 128, 2, 2>(who, p, s);
    return launch_tile<kFormatMxSplit66, kSwigluOfTwoSplit, 128, 128, 2, 2>(who, p, s);
  }
  if (terms == DEW_MOE_SECOND_TERM_E2M3) {
    if (forced_tile_rows == 256) return launch_tile<kFormatMxSplit6, kSwigluOfTwoSplit, 256, 128, 2, 2>(who, p, s);
    return launch_tile<kFormatMxSplit6, kSwigluOfTwoSplit, 128, 128, 2, 2>(who, p, s);
  }
  if (forced_tile_rows == 256) return launch_tile<kFormatMxSplit, kSwigluOfTwoSplit, 256, 128, 2, 2>(who, p, s);
  return launch_tile<kFormatMxSplit, kSwigluOfTwoSplit, 128, 128, 2, 2>(who, p, s);
}

}  // namespace dew

extern "C" int dew_moe_gateup_swiglu_split_out(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                                               const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up,
                                               void* hidden_split, uint8_t* hidden_scales, int32_t rows, void* stream) {
  return dew::gateup_split_out_of("dew_moe_gateup_swiglu_split_out", DEW_MOE_SECOND_TERM_E4M3, x_split, x_scale, gather, offsets, gate, up, hidden_split,
                                  hidden_scales, rows, stream, DEW_MOE_GATE_SILU, 0.0f);
}

extern "C" int dew_moe_gateup_swiglu_split_fp6_out(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                                                   const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up,
                                                   void* hidden_split, uint8_t* hidden_scales, int32_t rows, void* stream) {
  return dew::gateup_split_out_of("dew_moe_gateup_swiglu_split_fp6_out", DEW_MOE_SECOND_TERM_E2M3, x_split, x_scale, gather, offsets, gate, up,
                                  hidden_split, hidden_scales, rows, stream, DEW_MOE_GATE_SILU, 0.0f);
}

extern "C" int dew_moe_gateup_swiglu_split_e2m3_pair_out(const void* x_split, const int32_t* gather, const int32_t* offsets,
                                                         const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden_split,
                                                         uint8_t* hidden_scales, int32_t rows, void* stream) {
  return dew::gateup_split_out_of("dew_moe_gateup_swiglu_split_e2m3_pair_out", DEW_MOE_TERMS_E2M3_PAIR, x_split, nullptr, gather, offsets, gate,
                                  up, hidden_split, hidden_scales, rows, stream, DEW_MOE_GATE_SILU, 0.0f);
}

// ---- the SwiGLU expert MLP on split rows as one call -----------------------------------------------------------------

extern "C" int dew_moe_prefers_split_rows(const dew_moe_bank* gate, const dew_moe_bank* up, const dew_moe_bank* down, int32_t rows) {
  using namespace dew;
  auto wants = [rows](const dew_moe_bank* bank) {
    return bank && bank->layout == DEW_MOE_LAYOUT_PREPARED && bank->format == DEW_MOE_W_MXFP4 && bank->width % 256 == 0 &&
           bank->depth % 128 == 0 && bank->experts >= 1 && rows / bank->experts >= DEW_MOE_SPLIT_ROWS_FROM;
  };
  return wants(gate) && wants(up) && wants(down) && gate->experts == up->experts && gate->depth == up->depth &&
                 gate->width == up->width && down->experts == gate->experts && down->depth == gate->width &&
                 down->depth <= kMaxBlockScaleDepth
             ? 1
             : 0;
}

namespace dew {

struct SplitMlpWorkspace {
  size_t offsets, x_split, x_scale, hidden_split, hidden_scales, bytes;
};

static SplitMlpWorkspace split_mlp_workspace(int64_t tokens, int64_t rows, int64_t depth, int64_t hidden_width, int64_t experts) {
  auto rounded = [](size_t bytes) { return (bytes + 255) / 256 * 256; };
  SplitMlpWorkspace w{};
  size_t at = 0;
  w.offsets = at, at += rounded(static_cast<size_t>(experts + 1) * sizeof(int32_t));
  w.x_split = at, at += rounded(static_cast<size_t>(tokens) * depth * 2);
  w.x_scale = at, at += rounded(static_cast<size_t>(tokens));
  w.hidden_split = at, at += rounded(static_cast<size_t>(rows) * hidden_width * 2);
  w.hidden_scales = at, at += rounded(static_cast<size_t>(rows) * block_scale_pitch(static_cast<int>(hidden_width)));
  w.bytes = at + 256;  // room to align the caller's base
  return w;
}

}  // namespace dew

extern "C" size_t dew_moe_swiglu_mlp_split_workspace_bytes(int32_t tokens, int32_t rows, int32_t depth, int32_t hidden_width,
                                                           int32_t experts) {
  if (tokens < 0 || rows < 0 || depth < 0 || hidden_width < 0 || experts < 0) return 0;
  return dew::split_mlp_workspace(tokens, rows, depth, hidden_width, experts).bytes;
}

extern "C" int dew_moe_swiglu_mlp_split(const void* x, int32_t tokens, const int32_t* gather, const int32_t* offsets,
                                        const int32_t* group_sizes, const dew_moe_bank* gate, const dew_moe_bank* up,
                                        const dew_moe_bank* down, const int32_t* scatter, void* out, int32_t rows,
                                        int32_t second_term, void* workspace, size_t workspace_bytes, void* stream) {
  return dew_moe_gated_mlp_split(x, tokens, gather, offsets, group_sizes, gate, up, down, DEW_MOE_GATE_SILU, 0.0f, scatter, out, rows,
                                 second_term, workspace, workspace_bytes, stream);
}

extern "C" int dew_moe_gated_mlp_split(const void* x, int32_t tokens, const int32_t* gather, const int32_t* offsets,
                                       const int32_t* group_sizes, const dew_moe_bank* gate, const dew_moe_bank* up,
                                       const dew_moe_bank* down, int32_t activation, float limit, const int32_t* scatter, void* out,
                                       int32_t rows, int32_t second_term, void* workspace, size_t workspace_bytes, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_gated_mlp_split";
  if (int rc = check_bank(who, gate, "gate")) return rc;
  if (int rc = check_bank(who, up, "up")) return rc;
  if (int rc = check_bank(who, down, "down")) return rc;
  DEW_REQUIRE(tokens >= 0 && rows >= 0, "%s: tokens %d rows %d", who, tokens, rows);
  DEW_REQUIRE(second_term == DEW_MOE_SECOND_TERM_E4M3 || second_term == DEW_MOE_SECOND_TERM_E2M3 || second_term == DEW_MOE_TERMS_E2M3_PAIR,
              "%s: the rows' terms %d are neither two e4m3 (0), e4m3 and e2m3 (1) nor two e2m3 (2)", who, second_term);
  DEW_REQUIRE(down->experts == gate->experts && down->depth == gate->width, "%s: down [%d, %d, %d] does not follow gate [%d, %d, %d]", who,
              down->experts, down->depth, down->width, gate->experts, gate->depth, gate->width);
  if (rows == 0 || tokens == 0) return DEW_MOE_OK;
  DEW_REQUIRE((offsets != nullptr) != (group_sizes != nullptr), "%s: the groups come as offsets [E + 1] or as group_sizes [E], one of them", who);
  DEW_REQUIRE(gather != nullptr || rows <= tokens, "%s: %d rows of %d tokens need a gather", who, rows, tokens);
  const SplitMlpWorkspace w = split_mlp_workspace(tokens, rows, gate->depth, gate->width, gate->experts);
  DEW_REQUIRE(workspace && workspace_bytes >= w.bytes, "%s: workspace of %zu bytes, need %zu (dew_moe_swiglu_mlp_split_workspace_bytes)", who,
              workspace_bytes, w.bytes);
  uint8_t* base = reinterpret_cast<uint8_t*>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~static_cast<uintptr_t>(255));
  if (group_sizes != nullptr) {
    int32_t* formed = reinterpret_cast<int32_t*>(base + w.offsets);
    if (int rc = dew_moe_group_offsets(group_sizes, gate->experts, formed, stream)) return rc;
    offsets = formed;
  }
  void* x_split = base + w.x_split;
  uint8_t* x_scale = base + w.x_scale;
  void* hidden_split = base + w.hidden_split;
  uint8_t* hidden_scales = base + w.hidden_scales;
  if (second_term == DEW_MOE_TERMS_E2M3_PAIR) {
    if (int rc = dew_moe_split_rows_e2m3_pair(x, x_split, tokens, gate->depth, stream)) return rc;
  } else if (second_term == DEW_MOE_SECOND_TERM_E2M3) {
    if (int rc = dew_moe_split_rows_fp6(x, x_split, x_scale, tokens, gate->depth, stream)) return rc;
  } else {
    if (int rc = dew_moe_split_rows(x, x_split, x_scale, tokens, gate->depth, stream)) return rc;
  }
  if (int rc = gateup_split_out_of(who, second_term, x_split, x_scale, gather, offsets, gate, up, hidden_split, hidden_scales, rows, stream,
                                   activation, limit)) return rc;
  return dew_moe_grouped_gemm_split_blocks(hidden_split, hidden_scales, nullptr, offsets, down, nullptr, scatter, out, rows, stream);
}

extern "C" int dew_moe_gateup_interleaved(const void* x, const int32_t* gather, const int32_t* offsets,
                                          const dew_moe_bank* gate_up, const float* bias, float limit, void* hidden,
                                          int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_gateup_interleaved";
  if (int rc = check_bank(who, gate_up, "gate_up")) return rc;
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  DEW_REQUIRE(limit > 0.0f, "%s: the clamp limit %g must be positive", who, static_cast<double>(limit));
  if (rows == 0) return DEW_MOE_OK;
  GemmParams p{};
  if (int rc = fill_single(who, p, x, gather, offsets, gate_up, bias, nullptr, hidden, rows)) return rc;
  p.round_bias = 1;
  p.limit = limit;
  return launch<kInterleavedGated>(who, p, gate_up->format, static_cast<hipStream_t>(stream));
}

static int gateup_swiglu_of(const char* who, const void* x, const int32_t* gather, const int32_t* offsets, const int32_t* sizes,
                            const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden, int32_t rows, void* stream,
                            int32_t activation = DEW_MOE_GATE_SILU, float limit = 0.0f) {
  using namespace dew;
  DEW_REQUIRE(activation == DEW_MOE_GATE_SILU || activation == DEW_MOE_GATE_GELU_TANH,
              "%s: the gate's activation %d is neither silu (0: swiglu) nor the tanh gelu (1: geglu)", who, activation);
  DEW_REQUIRE(limit >= 0.0f, "%s: the clamp limit %g must be positive (0: none)", who, static_cast<double>(limit));
  if (int rc = check_bank(who, gate, "gate")) return rc;
  if (int rc = check_bank(who, up, "up")) return rc;
  DEW_REQUIRE(gate->format == up->format && gate->experts == up->experts && gate->depth == up->depth && gate->width == up->width,
              "%s: gate [%d, %d, %d] format %d and up [%d, %d, %d] format %d differ", who, gate->experts, gate->depth,
              gate->width, gate->format, up->experts, up->depth, up->width, up->format);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(x && (offsets || sizes) && hidden, "%s: x, the groups' offsets (or sizes) and hidden must not be null", who);
  DEW_REQUIRE(aligned16(x) && aligned16(hidden), "%s: x and hidden must be 16-byte aligned", who);
  GemmParams p{};
  p.x = static_cast<const bf16_t*>(x);
  p.gather = gather;
  p.offsets = offsets;
  p.sizes = sizes;
  p.scatter = nullptr;
  p.w0 = BankView{static_cast<const uint8_t*>(gate->codes), gate->scales, gate->tensor_scale};
  p.w1 = BankView{static_cast<const uint8_t*>(up->codes), up->scales, up->tensor_scale};
  p.out = static_cast<bf16_t*>(hidden);
  p.experts = gate->experts;
  p.depth = gate->depth;
  p.width = gate->width;
  p.rows = rows;
  p.gating = activation;
  p.limit = limit > 0.0f ? bf16_round_host(limit) : 0.0f;  // the clamp is compared in the operands' dtype
  return launch<kSwigluOfTwo>(who, p, gate->format, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_gateup_gated_f16(const void* x_f16, const uint8_t* x_scale, const int32_t* gather, const int32_t* offsets,
                                        const int32_t* group_sizes, const dew_moe_bank* gate, const dew_moe_bank* up, int32_t activation,
                                        float limit, void* hidden, int32_t rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_gateup_gated_f16";
  DEW_REQUIRE(activation == DEW_MOE_GATE_SILU || activation == DEW_MOE_GATE_GELU_TANH,
              "%s: the gate's activation %d is neither silu (0: swiglu) nor the tanh gelu (1: geglu)", who, activation);
  DEW_REQUIRE(limit >= 0.0f, "%s: the clamp limit %g must be positive (0: none)", who, static_cast<double>(limit));
  if (int rc = check_bank(who, gate, "gate")) return rc;
  if (int rc = check_bank(who, up, "up")) return rc;
  DEW_REQUIRE(gate->format == DEW_MOE_W_NVFP4 && up->format == DEW_MOE_W_NVFP4,
              "%s: f16 rows multiply NVFP4 banks whose block scales carry mantissas (an MXFP4 bank's power-of-two scales cost "
              "nothing on bf16 rows: dew_moe_gateup_gated); these are formats %d and %d", who, gate->format, up->format);
  DEW_REQUIRE(gate->experts == up->experts && gate->depth == up->depth && gate->width == up->width,
              "%s: gate [%d, %d, %d] and up [%d, %d, %d] differ", who, gate->experts, gate->depth, gate->width, up->experts, up->depth,
              up->width);
  DEW_REQUIRE(rows >= 0, "%s: rows %d", who, rows);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE((offsets != nullptr) != (group_sizes != nullptr), "%s: the groups come as offsets [E + 1] or as group_sizes [E], one of them", who);
  DEW_REQUIRE(x_f16 && x_scale && hidden, "%s: x_f16, x_scale and hidden must not be null", who);
  DEW_REQUIRE(aligned16(x_f16) && aligned16(hidden), "%s: x_f16 and hidden must be 16-byte aligned", who);
  GemmParams p{};
  p.x = static_cast<const bf16_t*>(x_f16);
  p.a_scale = x_scale;
  p.gather = gather;
  p.offsets = offsets;
  p.sizes = group_sizes;
  p.w0 = BankView{static_cast<const uint8_t*>(gate->codes), gate->scales, gate->tensor_scale};
  p.w1 = BankView{static_cast<const uint8_t*>(up->codes), up->scales, up->tensor_scale};
  p.out = static_cast<bf16_t*>(hidden);
  p.experts = gate->experts;
  p.depth = gate->depth;
  p.width = gate->width;
  p.rows = rows;
  p.gating = activation;
  p.limit = limit > 0.0f ? bf16_round_host(limit) : 0.0f;
  return launch_format<kFormatNvF16, kSwigluOfTwo>(who, p, static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_gateup_gated(const void* x, const int32_t* gather, const int32_t* offsets, const int32_t* group_sizes,
                                    const dew_moe_bank* gate, const dew_moe_bank* up, int32_t activation, float limit,
                                    void* hidden, int32_t rows, void* stream) {
  using namespace dew;
  DEW_REQUIRE(rows == 0 || (offsets != nullptr) != (group_sizes != nullptr),
              "dew_moe_gateup_gated: the groups come as offsets [E + 1] or as group_sizes [E], one of them");
  return gateup_swiglu_of("dew_moe_gateup_gated", x, gather, offsets, group_sizes, gate, up, hidden, rows, stream, activation, limit);
}

extern "C" int dew_moe_gateup_swiglu(const void* x, const int32_t* gather, const int32_t* offsets,
                                     const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden, int32_t rows,
                                     void* stream) {
  return gateup_swiglu_of("dew_moe_gateup_swiglu", x, gather, offsets, nullptr, gate, up, hidden, rows, stream);
}

extern "C" int dew_moe_gateup_swiglu_sizes(const void* x, const int32_t* gather, const int32_t* group_sizes,
                                           const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden, int32_t rows,
                                           void* stream) {
  return gateup_swiglu_of("dew_moe_gateup_swiglu_sizes", x, gather, nullptr, group_sizes, gate, up, hidden, rows, stream);
}
