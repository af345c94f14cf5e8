/* C ABI of libdew_moe_hip.so: the MI355X (gfx950) kernels of the quantized Mixture-of-Experts expert path.
 *
 * Plain pointers and sizes only: every pointer is DEVICE memory on the current HIP device unless said
 * otherwise, `stream` is a hipStream_t passed as void*. No entry point allocates or frees, and none but the
 * load-time dew_moe_prepare_bank synchronizes:
 * group bookkeeping is read on the device from `offsets`, so calls are stream-ordered and graph-safe, as
 * the reference's CUTLASS FFI library is (kernels/cutlass/ffi.cu:1-6, groups.cuh:19-30). Every entry point
 * returns 0 on success and a nonzero DEW_MOE_E* code otherwise; dew_moe_last_error() then names the refused
 * argument, as the reference's `const char* why` does (kernels/cutlass/grouped.h:56-65, ffi.cu:93-95).
 *
 * Notation: T tokens, D model width, F expert hidden width, E experts, k choices a token, R = T*k routed
 * slots. bf16 tensors are row-major uint16 bit patterns.
 */
#ifndef DEW_MOE_HIP_H
#define DEW_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  DEW_MOE_OK = 0,
  DEW_MOE_EINVAL = 1,   /* a shape, alignment or null-pointer contract is not met            */
  DEW_MOE_EDEVICE = 2,  /* the current device is not gfx950 (ffi.cu:102-106 refuses by name)  */
  DEW_MOE_ELAUNCH = 3   /* hipGetLastError() after a launch                                   */
};

/* Weight formats (reference layouts; src/dew/nn/kernels/formats.py:27-47, src/dew/interop/codecs.py:670-703).
 * K = depth (inputs), N = width (outputs) of each expert's matrix W[e] : [K, N].                       */
enum {
  DEW_MOE_W_FP8_BLOCK = 1,   /* codes u8 e4m3 [E,K,N]; scales f32 [E,ceil(K/128),ceil(N/128)]           */
  DEW_MOE_W_FP8_CHANNEL = 2, /* codes u8 e4m3 [E,K,N]; scales f32 [E,N]                                 */
  DEW_MOE_W_NVFP4 = 3,       /* codes = NvFp4.words u32 [E,N,K/8] (staged order, GF(2)-encoded);        */
                             /* scales = NvFp4.scales e4m3 bytes [E,N,K/16]; tensor_scale f32 [E].      */
                             /* MXFP4 banks arrive in this form (codecs.mxfp4_as_nvfp4).                */
  DEW_MOE_W_MXFP4 = 4,       /* prepared banks only: an NVFP4 bank whose block scales are all powers of */
                             /* two, as an MXFP4 checkpoint's are; dew_moe_prepare_bank finds it so.    */
  DEW_MOE_W_MXFP8 = 5,       /* OCP MXFP8, K-major as `formats.MxFp8` holds a product's matrices: codes */
                             /* u8 e4m3 [E,N,K]; scales u8 e8m0 [E,N,K/32]. For dew_moe_grouped_gemm_   */
                             /* mxfp8_rows only.                                                        */
  DEW_MOE_W_BF16 = 6,        /* unquantized matrices as the reference holds them: codes bf16 [E,K,N]    */
                             /* (`experts/<name>_proj/kernel`, src/dew/nn/moe.py:1231-1235); no scales. */
                             /* With DEW_MOE_LAYOUT_REFERENCE_KMAJOR, codes bf16 [E,N,K]: the same memory    */
                             /* read as the transposed matrices (an input gradient's: depth and width   */
                             /* are then the transposed product's). In the plain layout K is any whole  */
                             /* number of 64s and N of 32s (GPT-OSS's 2880: the reference's kernel takes */
                             /* whole 8s, grouped_matmul.py:1874-1887), and so are a DEW_MOE_W_MXFP4_BLOCKS */
                             /* bank's; every other bank's are whole 128s (an NVFP4 bank's depth 256s).   */
  DEW_MOE_W_MXFP4_BLOCKS = 7 /* an MXFP4 checkpoint's own tensors, for dew_moe_prepare_bank only: codes =  */
                             /* `*_blocks` u8 [E,N,K/32,16] (low nibble the even element), scales =       */
                             /* `*_scales` E8M0 u8 [E,N,K/32] (src/dew/interop/codecs.py:193-224). The    */
                             /* prepared bank is DEW_MOE_W_MXFP4 (or _NVFP4) and holds its tensor scales. */
};
/* With DEW_MOE_LAYOUT_REFERENCE_KMAJOR a DEW_MOE_W_FP8_BLOCK bank is a DeepSeek-style checkpoint's own tensors stacked by
 * expert: codes = `weight` e4m3 [E,N,K] ([out, in]), scales = `weight_scale_inv` f32 [E,N/128,K/128]
 * (src/dew/interop/codecs.py:670-703).                                                                            */

enum { DEW_MOE_LAYOUT_REFERENCE = 0, DEW_MOE_LAYOUT_PREPARED = 1, DEW_MOE_LAYOUT_REFERENCE_KMAJOR = 2 };

typedef struct dew_moe_bank {
  int32_t format;            /* DEW_MOE_W_*                                                             */
  int32_t layout;            /* DEW_MOE_LAYOUT_*                                                        */
  int32_t experts, depth, width;
  const void* codes;
  const void* scales;
  const float* tensor_scale; /* NVFP4 only, else NULL                                                   */
} dew_moe_bank;

enum { DEW_MOE_SCORE_SOFTMAX = 0, DEW_MOE_SCORE_SIGMOID = 1,
       DEW_MOE_SCORE_SQRTSOFTPLUS = 2 /* DeepSeek V4's sqrt(softplus(logit)), src/dew/nn/moe.py:303-313, 539-540 */ };
enum { DEW_MOE_GROUP_TOP2 = 0, DEW_MOE_GROUP_MAX = 1 };  /* a group's score: its two best selections' sum, or its best (src/dew/nn/moe.py:557-565) */

/* A router's fixed description (the fields of `Router`, src/dew/nn/moe.py:316-465, that its arithmetic reads). */
typedef struct dew_moe_router {
  int32_t experts, top_k;
  int32_t score_function;  /* DEW_MOE_SCORE_*                                              */
  int32_t normalize;       /* normalize_weights                                            */
  float scaling;           /* routed_scaling_factor                                        */
  int32_t expert_groups, groups_per_token;
  int32_t group_score;     /* DEW_MOE_GROUP_*                                              */
  /* The switches below follow `Router`'s fields of the same names (src/dew/nn/moe.py:361-384, read at :483-494 and
   * :510-513). All zero but weight_sum_epsilon = DEW_MOE_WEIGHT_SUM_EPSILON is the router the fields above describe. */
  int32_t bias_in_weights;      /* LLaDA-MoE: the weights are the chosen scores + bias, not the chosen scores        */
  float weight_sum_epsilon;     /* added to the chosen weights' sum before a renormalization divides by it           */
  float weight_sum_min;         /* ERNIE 4.5's moe_norm_min: above 0, the least that sum (+ epsilon) divides by; a
                                 * softmax router then renormalizes its chosen scores this way too                   */
  int32_t fill_excluded;        /* whether excluded_group_score is set (else an excluded expert is never chosen)     */
  float excluded_group_score;   /* A.X-K2's 0.0: what an expert outside a token's best groups is chosen by           */
  float logit_softcap;          /* Laguna: above 0, every logit is read as cap * tanh(logit / cap); 0 for none       */
} dew_moe_router;
#define DEW_MOE_WEIGHT_SUM_EPSILON 1e-20f   /* WEIGHT_SUM_EPSILON, src/dew/nn/moe.py:181 */

/* ---- introspection (kernels/cutlass/ffi.cu:133-176: dew_cutlass_kernels/kernel_fields/architecture) ---- */
const char* dew_moe_last_error(void);   /* thread-local, valid until the thread's next failing call      */
const char* dew_moe_architecture(void); /* "gfx950"                                                      */
const char* dew_moe_kernels(void);      /* one line per kernel: name, tile, waves, MFMA instruction      */
const char* dew_moe_kernel_fields(void);
int dew_moe_device_check(void);         /* DEW_MOE_OK iff the current device is gfx950                    */

/* ---- Router (src/dew/nn/moe.py:466-565, from the logits on) ----------------------------------------
 * scores = softmax | sigmoid of logits[T,E]; selection = scores (+ bias[E]); with expert_groups > 1 only the
 * experts of the groups_per_token best groups (a group's score = sum of its two best selections) stay,
 * the rest -inf; indices = the k largest selections in descending order, ties to the lower index;
 * weights = softmax of the chosen logits (softmax and normalize), else the chosen scores, divided by
 * (their sum + 1e-20) when normalize; times `scaling`. Bit-exact with the CPU oracle.                   */
int dew_moe_route(const float* logits, const float* bias /* nullable */, int32_t tokens, int32_t experts,
                  int32_t top_k, int32_t score_function, int32_t normalize, float scaling,
                  int32_t expert_groups, int32_t groups_per_token, float* weights /* [T,k] */,
                  int32_t* indices /* [T,k] */, void* stream);

/* dew_moe_route that also writes what the router sows for the balance statistics (src/dew/nn/moe.py:474-479): the
 * activated scores[T,E] and log_z[T] = logsumexp of the logits (either may be null).                            */
int dew_moe_route_sown(const float* logits, const float* bias /* nullable */, int32_t tokens, int32_t experts,
                       int32_t top_k, int32_t score_function, int32_t normalize, float scaling,
                       int32_t expert_groups, int32_t groups_per_token, float* weights, int32_t* indices,
                       float* scores /* nullable [T,E] */, float* log_z /* nullable [T] */, void* stream);

/* dew_moe_route_sown from a router's description, which also carries the switches the two entry points above fix
 * (sqrtsoftplus scores, `group_score='max'`). scores and log_z may be null.                                       */
int dew_moe_route_with(const dew_moe_router* router /* host */, const float* logits, const float* bias /* nullable */,
                       int32_t tokens, float* weights, int32_t* indices, float* scores, float* log_z, void* stream);

/* dew_moe_route_with with the per-token inputs of `Router.__call__(x, tokens, media, routes)` (src/dew/nn/moe.py:466-524):
 *  - media [T] with media_bias [E] (both or neither): DeepSeek-V4.1's image-span tokens, whose experts are chosen by
 *    scores + media_bias in place of scores + bias (`selection`, :516-524);
 *  - given [T,k], covered [T] (`chosen_experts`, :202-224: a replayed record of an engine's routing; and the hash router's
 *    `tid2eid[token ids]`, :500-507): token t uses given[t, :] in that order in place of its own top-k, where `covered` is
 *    null or covered[t] != 0. An id outside [0, experts) (a dropped slot's sentinel in a record) is written to `indices` as
 *    it came, with weight 0 and no part in the token's other weights; dew_moe_permute puts such a slot in no group, so the
 *    products write its row as zeros, as the reference's sort drops it (`_sorted_locally`, :1101-1128).
 * The weights are the router's for the experts used (:483-494). All four null is dew_moe_route_with.                  */
int dew_moe_route_call(const dew_moe_router* router /* host */, const float* logits, const float* bias /* nullable */,
                       const float* media_bias /* nullable [E] */, const uint8_t* media /* nullable [T] */,
                       const int32_t* given /* nullable [T,k] */, const uint8_t* covered /* nullable [T] */,
                       int32_t tokens, float* weights, int32_t* indices, float* scores, float* log_z, void* stream);

/* LLaDA2.2's block routing (`routing_block` / `block_experts`, `Router.block_mask` src/dew/nn/moe.py:566-585, applied in
 * `selection` :516-524): the tokens are `rows` x `length`; blocks[t] numbers token t's block within its row from 0 (the
 * reference's `numbered_blocks`, src/dew/nn/inputs.py:462-476), negative for padding, which is a block of its own. A block's
 * score for an expert is its best token's selection (scores + bias); a token chooses its top_k among the `block_experts`
 * best of its block (ties to the lower index). Three launches and a clearing one on `stream`; the workspace
 * (dew_moe_route_blocks_workspace_bytes: a key per block and expert, a shortlist per block) is the caller's, no allocation
 * here. The router has no expert groups.                                                                                  */
size_t dew_moe_route_blocks_workspace_bytes(int32_t rows, int32_t length, int32_t experts);
int dew_moe_route_blocks(const dew_moe_router* router /* host */, const float* logits /* [rows * length, E] */,
                         const float* bias /* nullable */, const int32_t* blocks /* [rows * length] */, int32_t rows,
                         int32_t length, int32_t block_experts, void* workspace, size_t workspace_bytes, float* weights,
                         int32_t* indices, float* scores /* nullable */, float* log_z /* nullable */, void* stream);

/* The aux-loss-free balancing step (`load_balance_update` src/dew/nn/moe.py:271-300, applied to the selection bias as
 * `_updated_bias` src/dew/objectives/routing.py:342-345): bias[e] += rate * direction, direction -1 where counts[e]
 * is above floor(sum / E), +1 where below it or equal with a remainder, else 0. counts = dew_moe_permute's sizes. */
int dew_moe_balance_bias(const int32_t* counts /* [E] */, float* bias /* [E], updated in place */, float rate,
                         int32_t experts, void* stream);

/* Gate logits (src/dew/nn/moe.py:526-534): logits[T,E] = f32(x[T,D] bf16) @ kernel[D,E] f32, IEEE fp32, plus
 * bias[E] where the router has one (GPT-OSS's, src/dew/nn/gpt_oss.py:163-165).                              */
int dew_moe_router_logits(const void* x /* bf16 [T,D] */, const float* kernel /* [D,E] */,
                          const float* bias /* nullable [E] */, float* logits /* [T,E] */, int32_t tokens,
                          int32_t depth, int32_t experts, void* stream);

/* ---- Dispatch bookkeeping (src/dew/nn/moe.py:1101-1128 `_sorted_locally`) --------------------------
 * Stable counting sort of the R = tokens*top_k flattened expert ids: sizes[E] = bincount,
 * offsets[E+1] = exclusive prefix (offsets[E] = number of slots whose id is < E), order[R] = argsort
 * (slot index of each sorted position; ids >= E sort last in slot order), rows[R] = order / top_k.       */
size_t dew_moe_permute_workspace_bytes(int32_t slots, int32_t experts);
int dew_moe_permute(const int32_t* indices /* [T,k] */, int32_t tokens, int32_t top_k, int32_t experts,
                    int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows, void* workspace,
                    size_t workspace_bytes, void* stream);

/* dew_moe_permute with an always-on (shared) expert folded in as group E (src/dew/nn/moe.py:1497-1503 adds the shared
 * expert's output to every token's; as one more group of the same grouped launches it costs no launch of its own):
 * behind the R routed slots come `shared_rows` more sorted positions, one a token, that belong to group E and read row
 * i of the activations: sizes[E + 1] (sizes[E] = shared_rows), offsets[E + 2], order[R + shared_rows] and
 * rows[R + shared_rows], with order = R + i and rows = i for the shared group's position i; dropped slots (ids outside
 * [0, E)) still sort last, behind the shared group. Workspace: dew_moe_permute_workspace_bytes(R + shared_rows, E + 1). */
int dew_moe_permute_shared(const int32_t* indices /* [T,k] */, int32_t tokens, int32_t top_k, int32_t experts,
                           int32_t shared_rows, int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows,
                           void* workspace, size_t workspace_bytes, void* stream);

/* dew_moe_permute for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc) and so have no workspace to hand in; no counterpart in the reference, whose FFI
 * handler takes its workspace from XLA's ScratchAllocator. The sort's per-block counts live in an array of
 * DEW_MOE_PERMUTE_STATIC_BYTES that the library itself holds on every GPU it runs on until the process ends; a
 * problem whose dew_moe_permute_workspace_bytes() is larger is refused (slots / 2048 blocks x (experts + 1) x 8 bytes:
 * 1 MiB covers e.g. 2^20 slots over 255 experts). Calls on one GPU share that array: calls that overlap on
 * different streams of one GPU race; calls in stream order need nothing cleared between them. The call allocates and
 * frees nothing; outputs are identical to dew_moe_permute's. The device the stream belongs to must be current: the
 * first call on a device looks up that device's copy of the array (hipGetSymbolAddress, once), so make that call
 * before a capture begins.                                                                                        */
#define DEW_MOE_PERMUTE_STATIC_BYTES ((size_t)1 << 20)
int dew_moe_permute_static(const int32_t* indices /* [T,k] */, int32_t tokens, int32_t top_k, int32_t experts,
                           int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows, void* stream);

/* Capacity dropping (`capacity_positions` src/dew/nn/moe.py:832-855, applied at :914-919): indices [sequences, length,
 * top_k]; within each sequence a slot's place in its expert's queue is its rank, in slot order, among the sequence's slots
 * of that expert; admitted = the id where the place is below `capacity`, else `experts` (the dropped slot's sentinel,
 * which dew_moe_permute sorts last and outside every group, and whose rows the products write as zeros). The host
 * computes capacity = int(max(ceil(length * top_k / experts) * capacity_factor, capacity_factor)).               */
int dew_moe_capacity_admit(const int32_t* indices, int32_t sequences, int32_t length, int32_t top_k, int32_t experts,
                           int32_t capacity, int32_t* admitted /* [sequences, length, top_k] */, void* stream);

/* offsets[E+1] = exclusive prefix of group sizes[E] (implicit in jax.lax.ragged_dot's group_sizes,
 * src/dew/nn/kernels/xla_products.py:86-115; explicit at src/dew/nn/moe.py:1172).                        */
int dew_moe_group_offsets(const int32_t* sizes, int32_t experts, int32_t* offsets, void* stream);

/* ---- One-time weight re-layout -----------------------------------------------------------------------
 * The GEMM kernels read a bank re-laid into MFMA-fragment order (exact: a permutation of the codes; the
 * NVFP4 word encoder is an invertible GF(2) map, src/dew/algebra/bits.py:208-223,240-250). Call once per
 * bank at load; `prepared` must hold dew_moe_prepared_bytes() bytes, 256-byte aligned. `out` describes
 * the prepared bank and is what the GEMM entry points take. For an NVFP4 bank the call waits for the
 * stream once, to read back whether every block scale is a power of two (then out->format is
 * DEW_MOE_W_MXFP4 and the kernels convert codes and scale in one hardware instruction). A checkpoint's MXFP4
 * tensors (DEW_MOE_W_MXFP4_BLOCKS) become the same prepared bank as the reference's own conversion of them would
 * (`mxfp4_tensor_powers`, `mxfp4_as_nvfp4`, src/dew/interop/codecs.py:238-284, then `NvFp4.of`), without a value or a
 * word decoded; where the reference keeps such a bank dense (an expert's group powers spread past 17 binades, a 0xff
 * scale byte) the call refuses it by name. Load time only: the call synchronizes and is not for a captured step.  */
size_t dew_moe_prepared_bytes(int32_t format, int32_t experts, int32_t depth, int32_t width);
int dew_moe_prepare_bank(const dew_moe_bank* reference, void* prepared, dew_moe_bank* out /* host */,
                         void* stream);

/* The descriptor of a bank prepared earlier, from the buffer alone: for a binding that holds the prepared bytes as an
 * opaque array (an XLA buffer) and the bank's format tag and extents as static attributes. `format` is the PREPARED
 * bank's (out->format of dew_moe_prepare_bank); external_scales: a per-channel FP8 bank's f32 [E, N], else null;
 * tensor_scale: an FP4 bank's f32 [E] (for a bank prepared from DEW_MOE_W_MXFP4_BLOCKS, the ones that call wrote:
 * out->tensor_scale, which lies inside the prepared buffer), else null. Host only, no launch.                  */
int dew_moe_prepared_view(int32_t format, int32_t experts, int32_t depth, int32_t width, const void* prepared,
                          const void* external_scales, const float* tensor_scale, dew_moe_bank* out /* host */);

/* Tuning and testing knob (no counterpart in the reference): every later grouped product launched by the CALLING
 * THREAD uses block tiles of `rows` rows (32, 64, 128 or 256; 256 with FP4 banks whose width is whole 256s); 0, the
 * default, chooses per launch from the rows, experts and width. The setting is thread-local: other threads' launches
 * (an FFI thread pool's) keep their own choice.                                                              */
int dew_moe_tile_rows(int32_t rows);

/* ---- Grouped products (src/dew/nn/moe.py:666-770 expert_projection / paired_projections; replaces the
 *      launches of kernels/cutlass/ffi.cu:180-220 behind src/dew/nn/kernels/grouped_matmul.py:1826-1831) --
 * Sorted position i in [offsets[e], offsets[e+1]) belongs to expert e and reads row gather[i] of x (row i
 * when gather is NULL). out row = scatter[i] (i when NULL). Operands bf16, weights dequantized to bf16
 * exactly as the reference's load does, fp32 accumulation, one rounding to bf16. Sorted positions in
 * [offsets[E], rows) are written as zeros (kernels/cutlass/ffi.cu:117-123).                             */
int dew_moe_grouped_gemm(const void* x /* bf16 [*,K] */, const int32_t* gather, const int32_t* offsets,
                         const dew_moe_bank* w /* prepared, [E,K,N] */, const int32_t* scatter,
                         void* out /* bf16 [rows,N] */, int32_t rows, void* stream);

/* dew_moe_grouped_gemm_bias and dew_moe_gateup_swiglu taking the groups as the reference's FFI targets take them:
 * `group_sizes s32[E]`, the operand of jax.lax.ragged_dot and of dew_cutlass_grouped_gemm (kernels/cutlass/ffi.cu:180-198,
 * groups.cuh:19-30). The exclusive prefix is formed on the device inside each block's tile search, so a launch class
 * that holds sizes needs no prefix launch; everything else is the entry point of the same name without `_sizes`.   */
int dew_moe_grouped_gemm_sizes(const void* x, const int32_t* gather, const int32_t* group_sizes /* [E] */,
                               const dew_moe_bank* w, const float* bias /* nullable */, const int32_t* scatter, void* out,
                               int32_t rows, void* stream);
int dew_moe_gateup_swiglu_sizes(const void* x, const int32_t* gather, const int32_t* group_sizes /* [E] */,
                                const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden, int32_t rows, void* stream);
/* dew_moe_grouped_gemm_bias (groups as offsets or sizes, the other NULL) taking the bias as the parameter holds it, fp32: the
 * launch rounds it to the compute dtype as it reads it (`rounded_operand`, src/dew/nn/moe.py:729-742), so the caller
 * makes no rounding pass of its own a call. dew_moe_gateup_interleaved reads its bias the same way.             */
int dew_moe_grouped_gemm_param_bias(const void* x, const int32_t* gather, const int32_t* offsets /* nullable */,
                                    const int32_t* group_sizes /* nullable */, const dew_moe_bank* w, const float* bias,
                                    const int32_t* scatter, void* out, int32_t rows, void* stream);

/* The same with each expert's bias[E,N] (values of the compute dtype held in fp32) added to its rows' fp32
 * sums before their one rounding (src/dew/nn/moe.py:729-742 _biased / _plus_bias; NULL = none).          */
int dew_moe_grouped_gemm_bias(const void* x, const int32_t* gather, const int32_t* offsets,
                              const dew_moe_bank* w, const float* bias, const int32_t* scatter, void* out,
                              int32_t rows, void* stream);

/* GPT-OSS's fused gate_up bank, gate in the even columns and up in the odd ones, with its epilogue
 * (src/dew/nn/gpt_oss.py:111-121): projected = bf16(sum + bias), gate = min(even, limit), up = clip(odd,
 * +-limit), hidden[rows, N/2] = (up + 1) * gate * logistic(1.702 gate), every operation rounded to bf16 as
 * the reference's bf16 arrays round it.                                                                  */
int dew_moe_gateup_interleaved(const void* x, const int32_t* gather, const int32_t* offsets,
                               const dew_moe_bank* gate_up /* prepared, [E,K,2F] */, const float* bias /* nullable [E,2F] */,
                               float limit, void* hidden /* bf16 [rows,F] */, int32_t rows, void* stream);

/* Activation rows as two FP8 (e4m3) terms for the scaled matrix instructions (no counterpart in the reference:
 * its products take bf16 operands, src/dew/nn/moe.py:675-677, and this keeps their values): x = s (hi + lo / 16)
 * with s = 2^(scale[row] - 127) one power of two per row, exact for every element within 2^-11 of its row's
 * largest magnitude and to 2^-21 of that magnitude otherwise. split[row] holds each 64 depths as four 32-byte
 * pieces in the scaled instruction's operand order (hi then lo of depths 0-15 and 32-47, hi then lo of depths
 * 16-31 and 48-63): depth * 2 bytes a row, like the bf16 source.                                            */
int dew_moe_split_rows(const void* x /* bf16 [rows, depth] */, void* split /* [rows, depth * 2] bytes */,
                       uint8_t* scale /* [rows] e8m0 */, int32_t rows, int32_t depth, void* stream);

/* The grouped products on rows split by dew_moe_split_rows, for MXFP4 banks (every block scale a power of two,
 * DEW_MOE_W_MXFP4 after dew_moe_prepare_bank) whose width is whole 256s: v_mfma_scale_f32_32x32x64_f8f6f4 multiplies
 * each e4m3 term by the FP4 codes as stored, under both operands' power-of-two scales, so no weight is dequantized
 * and every product is the exact bf16 x weight product of dew_moe_grouped_gemm_bias / dew_moe_gateup_swiglu; only
 * the order of the fp32 sums differs. 256-row tiles: meant for groups of several hundred rows.            */
int dew_moe_grouped_gemm_split(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                               const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                               const int32_t* scatter, void* out, int32_t rows, void* stream);
int dew_moe_gateup_swiglu_split(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                                const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up,
                                void* hidden, int32_t rows, void* stream);
/* The pair that keeps the whole expert MLP on the scaled instruction without a split pass between its products:
 * the gate/up launch writes its SwiGLU rows already split, two e4m3 terms under one scale per row and 128 columns
 * (hidden_split [rows, F * 2] bytes in dew_moe_split_rows' order; hidden_scales [rows, P] e8m0 bytes, byte b of a
 * row the scale of its columns 128 b .. 128 b + 127, with P = F / 128 rounded up to a multiple of 16 and the base
 * 16-byte aligned; the values are the bf16 hidden rows of dew_moe_gateup_swiglu, exactly, within 2^-11 of each
 * block's largest magnitude), and the down launch reads rows split that way (x_scales [source rows, P of K]; K up to
 * 24576: a tile keeps its rows' scales in the LDS).                                                              */
int dew_moe_gateup_swiglu_split_out(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                                    const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up,
                                    void* hidden_split, uint8_t* hidden_scales, int32_t rows, void* stream);
int dew_moe_grouped_gemm_split_blocks(const void* x_split, const uint8_t* x_scales, const int32_t* gather,
                                      const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                                      const int32_t* scatter, void* out, int32_t rows, void* stream);

/* The SwiGLU expert MLP on split rows as one call (`ExpertMLP._project`, src/dew/nn/moe.py:1305-1326: paired gate/up
 * products, `gated_product('swiglu')`, the down product): dew_moe_split_rows (or _fp6) of x[tokens, D], then
 * dew_moe_gateup_swiglu_split_out and dew_moe_grouped_gemm_split_blocks, the split rows and the split hidden rows in
 * `workspace` (dew_moe_swiglu_mlp_split_workspace_bytes; any alignment). The groups come as `offsets [E + 1]` or as
 * `group_sizes [E]` (the reference FFI's operand, kernels/cutlass/ffi.cu:185-198), the other null. out is bf16 [rows, down
 * width], row i at scatter[i] where scatter is given. dew_moe_prefers_split_rows is the rule by which the host mirror takes
 * this form (1) or the bf16-operand launches (0): three prepared MXFP4 banks of whole 256-column strips that chain, the
 * down bank's depth within the LDS's room for a tile's scales, and groups averaging DEW_MOE_SPLIT_ROWS_FROM rows or more
 * (measured: 1.20 times the bf16 launches at 900 rows a group, 1.05 at 512 to 768, 1.08 at 384, 0.975 at 256).       */
enum { DEW_MOE_SECOND_TERM_E4M3 = 0, DEW_MOE_SECOND_TERM_E2M3 = 1, DEW_MOE_TERMS_E2M3_PAIR = 2 /* both terms e2m3, below */ };
#define DEW_MOE_SPLIT_ROWS_FROM 384
int dew_moe_prefers_split_rows(const dew_moe_bank* gate, const dew_moe_bank* up, const dew_moe_bank* down, int32_t rows);
size_t dew_moe_swiglu_mlp_split_workspace_bytes(int32_t tokens, int32_t rows, int32_t depth, int32_t hidden_width, int32_t experts);
int dew_moe_swiglu_mlp_split(const void* x /* bf16 [tokens, D] */, int32_t tokens, const int32_t* gather /* nullable [rows] */,
                             const int32_t* offsets /* [E + 1] or null */, const int32_t* group_sizes /* [E] or null */,
                             const dew_moe_bank* gate, const dew_moe_bank* up, const dew_moe_bank* down,
                             const int32_t* scatter /* nullable [rows] */, void* out, int32_t rows,
                             int32_t second_term /* DEW_MOE_SECOND_TERM_* */, void* workspace, size_t workspace_bytes, void* stream);
/* The same with the gate the experts name (`activation` = DEW_MOE_GATE_*, below: SwiGLU or GeGLU) and, where `limit` is
 * positive, `swiglu_clamped`'s clamp of both products before it (src/dew/nn/activations.py:327-356): clamped or GeGLU experts
 * on MXFP4 banks stay on split rows; dew_moe_swiglu_mlp_split is this with SwiGLU and no clamp.                          */
int dew_moe_gated_mlp_split(const void* x, int32_t tokens, const int32_t* gather, const int32_t* offsets, const int32_t* group_sizes,
                            const dew_moe_bank* gate, const dew_moe_bank* up, const dew_moe_bank* down, int32_t activation,
                            float limit, const int32_t* scatter, void* out, int32_t rows, int32_t second_term, void* workspace,
                            size_t workspace_bytes, void* stream);

/* EXPERIMENTAL options (this one and the next): not exact, outside the 2e-2 element-wise bar the default launches hold
 * (a 512-deep MLP has read 2.1e-2; the reference's own metric max|d| / max|ref| stays under 1e-2), off by default everywhere.
 * The first product of that pair with the rows' second term in FP6 (no counterpart in the reference). dew_moe_split_rows_fp6:
 * x = s hi + t lo with hi = e4m3(x / s) under one power-of-two scale s a row (scale[row], as dew_moe_split_rows) and
 * lo = e2m3((x - s hi) / t) under t, one power of two for every 32 depths. Each 64 depths of a row are 128 bytes: for
 * lane group g = 0, 1: 32 bytes of hi codes (depths 16 g .. 16 g + 15, then 32 + 16 g .. 47 + 16 g), 24 bytes of lo codes
 * (depths 32 g .. 32 g + 31, six bits each, in order), t's e8m0 byte in a dword, 4 unused bytes. The second term's
 * instruction (FP6 x FP4) takes half the cycles of the first's, so the launch runs faster than on two e4m3 terms; the
 * price is that an element more than two binades below its 32-deep block's largest magnitude is held to within 2^-10 of
 * that magnitude, not exactly (dew_moe_split_rows: exactly within 2^-11 of the ROW's largest).
 * dew_moe_gateup_swiglu_split_fp6_out is dew_moe_gateup_swiglu_split_out on such rows; its hidden rows leave in that
 * entry point's format (two e4m3 terms under a scale per row and 128 columns).                                   */
int dew_moe_split_rows_fp6(const void* x /* bf16 [rows, depth] */, void* split /* [rows, depth * 2] bytes */,
                           uint8_t* scale /* [rows] e8m0 */, int32_t rows, int32_t depth, void* stream);
int dew_moe_gateup_swiglu_split_fp6_out(const void* x_split, const uint8_t* x_scale, const int32_t* gather,
                                        const int32_t* offsets, const dew_moe_bank* gate, const dew_moe_bank* up,
                                        void* hidden_split, uint8_t* hidden_scales, int32_t rows, void* stream);

/* The same first product with BOTH terms in FP6 (no counterpart in the reference; an option, not the default, for the same
 * reason as the FP6 second term: it is not exact). dew_moe_split_rows_e2m3_pair: x = s hi + t lo, hi = e2m3(x / s),
 * lo = e2m3((x - s hi) / t), s and t each one power of two for every 32 depths (the least that brings the block's largest
 * magnitude, then its largest remainder, within 7.5); no scale a row. Each 64 depths of a row are 128 bytes: for lane group
 * g = 0, 1 (depths 32 g .. 32 g + 31): 24 bytes of hi codes (six bits each, in order), s's e8m0 byte in a dword, 4 unused
 * bytes, then the same for lo and t. An element within two binades of its block's largest magnitude is held exactly, any
 * other to within 2^-10 of that magnitude: the bound of dew_moe_split_rows_fp6, whose launch this one replaces at two
 * thirds of its matrix-instruction time (two FP6 x FP4 instructions: the time of ONE FP8 x FP4 instruction).
 * dew_moe_gateup_swiglu_split_e2m3_pair_out is dew_moe_gateup_swiglu_split_out on such rows (no x_scale); its hidden rows
 * leave as two e4m3 terms under a scale per row and 128 columns, as that entry point's do.                          */
int dew_moe_split_rows_e2m3_pair(const void* x /* bf16 [rows, depth] */, void* split /* [rows, depth * 2] bytes */, int32_t rows,
                                 int32_t depth, void* stream);
int dew_moe_gateup_swiglu_split_e2m3_pair_out(const void* x_split, const int32_t* gather, const int32_t* offsets,
                                              const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden_split,
                                              uint8_t* hidden_scales, int32_t rows, void* stream);

/* The blockwise FP8 recipe's forward product (DeepSeek-V3's 1 x 128 activation tiles, 128 x 128 weight blocks):
 * `rows_quantized` src/dew/nn/kernels/projections.py:176-182 and `blockwise_fp8_product`
 * src/dew/nn/kernels/gemm.py:764-793 (its portable sum: `step_scaled` src/dew/nn/kernels/xla_products.py:147-173).
 * dew_moe_quantize_rows_fp8: x bf16 [rows, K] -> e4m3 codes a 1 x 128 tile at a time, amax floored at 1e-4, scale the
 * least power of two >= amax * f32(1 / 448) (src/dew/nn/fake_quant.py:117-128). codes [rows, K] bytes hold each 128
 * depths in the scaled matrix instruction's operand order: byte 16 (4 g + 2 t + h) + b is depth 64 t + 32 h + 16 g + b;
 * scales [rows, P] are the scales' e8m0 bytes (value 2^(byte - 127)), P = K / 128 rounded up to a multiple of 16.
 * dew_moe_grouped_gemm_fp8_rows: out[scatter[i]] = bf16( sum over 128-deep blocks of (codes x codes, exact) x row
 * scale x weight block scale (+ bias) ) for an FP8 128 x 128 block bank (prepared) whose scales are powers of two, as
 * the recipe's `blocks_quantized` makes them: both operands enter v_mfma_scale_f32_32x32x64_f8f6f4 as stored. A weight
 * block scale that is no normal power of two makes the tiles that meet it NaN. K up to 24576, rows in 256-row tiles. */
/* The MXFP8 recipe's forward product (OCP MX: e4m3 codes, one power-of-two E8M0 scale every 32 depths of both
 * operands): `MxFp8.quantized` src/dew/nn/kernels/formats.py:186-229 and `mxfp8_product`
 * src/dew/nn/kernels/gemm.py:882-892. dew_moe_quantize_rows_mxfp8: x bf16 [rows, K] -> codes [rows, K] bytes in the
 * operand order of dew_moe_quantize_rows_fp8 and scales [rows, K / 32] E8M0 bytes in depth order (scale = 2^(largest
 * magnitude's exponent - 8), byte 0 for a block of zeros; codes saturate at +-448). dew_moe_grouped_gemm_mxfp8_rows:
 * out[scatter[i]] = bf16( sum of exact (code x scale) products (+ bias) ) with a DEW_MOE_W_MXFP8 bank (prepared):
 * v_mfma_scale_f32_32x32x64_f8f6f4 takes the codes and the per-32 scales of both operands as they are stored, which
 * is the instruction's own format. K whole 128s, N whole 128s, rows in 256-row tiles.                           */
int dew_moe_quantize_rows_mxfp8(const void* x /* bf16 [rows, K] */, void* codes /* [rows, K] bytes */,
                                uint8_t* scales /* [rows, K / 32] e8m0 */, int32_t rows, int32_t depth, void* stream);
int dew_moe_grouped_gemm_mxfp8_rows(const void* x_codes, const uint8_t* x_scales, const int32_t* gather,
                                    const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                                    const int32_t* scatter, void* out, int32_t rows, void* stream);
/* The recipes' kernel gradients: each group's tokens contracted, out[g] = x[group g's tokens]^T @ dy[group g's
 * tokens] -> [groups, K, N]. Blockwise FP8: `_projection_backward` src/dew/nn/kernels/projections.py:211-224
 * (`rows_quantized(x.T)`, `rows_quantized(cotangent.T)`) and `blockwise_fp8_kernel_gradient`
 * src/dew/nn/kernels/gemm.py:795-819 (each 128-token block's exact partial times its rows' and columns' scales, fp32
 * sums; the recipe's scales are powers of two, taken here as E8M0 bytes). MXFP8: `_mx_backward`
 * src/dew/nn/kernels/projections.py:263-275 (`MxFp8.quantized(x.T)`, every 32 tokens a scale; the reference multiplies
 * the decoded operands in bf16 with fp32 sums, `gemm_t` src/dew/nn/kernels/gemm.py:418-431, which the scaled products
 * equal term for term).
 * dew_moe_quantize_columns_fp8 / _mxfp8: x bf16 [tokens, dim] quantized along the TOKENS (1 x 128 tiles under
 * dew_moe_quantize_rows_fp8's scale rule, or 32-token MX blocks under dew_moe_quantize_rows_mxfp8's) and written
 * transposed. as_bank 0 (the lhs_t operand): codes [dim, tokens] bytes in the row operand's order within each 128
 * tokens, scales [dim, tokens / 32] E8M0 bytes (the FP8 tile's byte repeated for its four 32s). as_bank 1 (the rhs_t
 * operand): the layout of a prepared DEW_MOE_W_MXFP8 bank of one expert, depth = tokens, width = dim: codes
 * [dim / 32][tokens / 32][64][16] bytes, then scales [dim / 32][tokens / 128][32][4]; wrap them in a dew_moe_bank
 * {MXFP8, PREPARED, experts 1, depth tokens, width dim}. tokens whole 128s (a recipe pads each group to them), dim
 * whole 128s.
 * dew_moe_kernel_gradient_mxfp8: out [groups, depth, width] (bf16, or fp32 where out_is_f32) from the lhs_t operand
 * [depth, tokens] and the rhs_t bank [width, tokens]; group g contracts tokens offsets[g] .. offsets[g + 1], whole
 * 128-token blocks (device int32 [groups + 1]); an empty group's matrix is zero. Both operands enter
 * v_mfma_scale_f32_32x32x64_f8f6f4 as stored, 256 x 256 tiles.                                                    */
int dew_moe_quantize_columns_fp8(const void* x /* bf16 [tokens, dim] */, void* codes, void* scales, int32_t tokens,
                                 int32_t dim, int32_t as_bank, void* stream);
int dew_moe_quantize_columns_mxfp8(const void* x /* bf16 [tokens, dim] */, void* codes, void* scales, int32_t tokens,
                                   int32_t dim, int32_t as_bank, void* stream);
int dew_moe_kernel_gradient_mxfp8(const void* lhs_t_codes, const uint8_t* lhs_t_scales, const dew_moe_bank* rhs_t,
                                  const int32_t* offsets, void* out, int32_t out_is_f32, int32_t depth, int32_t groups,
                                  void* stream);
/* The kernel gradient of bf16 operands: the reference's `gemm_t` src/dew/nn/kernels/gemm.py:418-431 (each group's rows
 * of lhs transposed times its rows of rhs, fp32 sums), and with it the NVFP4 recipe's `_nvfp4_backward`
 * src/dew/nn/kernels/projections.py:322-337 (both operands quantized along the tokens, every 16 a scale, decoded, the
 * tensor scales applied).
 * dew_moe_transpose_columns: x bf16 [tokens, dim] -> the lhs_t operand, rows [dim, tokens] bf16 (as_bank 0), or the
 * rhs_t operand in the layout of a prepared DEW_MOE_W_BF16 bank of one expert, depth = tokens, width = dim (as_bank 1:
 * atoms [dim / 32][tokens / 16][64][8 bf16]). dew_moe_quantize_columns_nvfp4: the same with every value replaced by its
 * NVFP4 value short of the tensor scale (E2M1 code x the E4M3 scale of its 16 tokens; dew_moe_quantize_rows_nvfp4's
 * arithmetic along the tokens) and *tensor_scale written; workspace is 4 bytes of device memory.
 * dew_moe_kernel_gradient_bf16: out [groups, depth, width] (bf16, or fp32 where out_is_f32) = lhs_t[:, tokens of g] x
 * rhs_t[:, tokens of g]^T, exact products, fp32 sums, times *lhs_scale x *rhs_scale (device floats, each may be null),
 * one rounding. Group g contracts tokens offsets[g] .. offsets[g + 1], whole 64-token steps. 256 x 256 tiles.        */
int dew_moe_transpose_columns(const void* x /* bf16 [tokens, dim] */, void* out, int32_t tokens, int32_t dim,
                              int32_t as_bank, void* stream);
/* dew_moe_transpose_groups: dew_moe_transpose_columns for ragged groups (`gemm_t`'s `group_sizes` are any sizes): x bf16
 * [rows, dim], group g its rows offsets[g] .. offsets[g + 1] (device int32 [groups + 1]); each group is written from a
 * whole 64-token step on and its last step filled with zeros, into padded_tokens tokens (whole 128s, at least rows +
 * 64 * groups; the rest zeros); padded_offsets [groups + 1] receives the groups' offsets in the written order, which
 * are dew_moe_kernel_gradient_bf16's. At most 4096 groups.                                                        */
int dew_moe_transpose_groups(const void* x /* bf16 [rows, dim] */, const int32_t* offsets, void* out,
                             int32_t* padded_offsets, int32_t rows, int32_t padded_tokens, int32_t dim, int32_t groups,
                             int32_t as_bank, void* stream);
int dew_moe_quantize_columns_nvfp4(const void* x /* bf16 [tokens, dim] */, void* values, float* tensor_scale,
                                   uint32_t* workspace, int32_t tokens, int32_t dim, int32_t as_bank, void* stream);
int dew_moe_kernel_gradient_bf16(const void* lhs_t, const dew_moe_bank* rhs_t, const int32_t* offsets,
                                 const float* lhs_scale, const float* rhs_scale, void* out, int32_t out_is_f32,
                                 int32_t depth, int32_t groups, void* stream);
/* The NVFP4 recipe's rows (`NvFp4Block.quantized` src/dew/nn/kernels/formats.py:263-274 over `bits.nvfp4_coded`
 * src/dew/algebra/bits.py:941-982): E2M1 codes under an E4M3 scale every 16 depths and one tensor scale (the
 * operand's largest magnitude over 6 x 448). The instruction has no such operand (its block scales are powers of two
 * over 32 depths), so the rows are written as the bf16 values they stand for short of the tensor scale (code x block
 * scale, exact in bf16) and multiplied by the NVFP4 bank through dew_moe_grouped_gemm with the two tensor scales'
 * product as the bank's (`nvfp4_block_product` src/dew/nn/kernels/gemm.py:937-947). workspace: 4 bytes of device
 * memory; tensor_scale: one device float, written.                                                               */
int dew_moe_quantize_rows_nvfp4(const void* x /* bf16 [rows, K] */, void* values /* bf16 [rows, K] */,
                                float* tensor_scale, uint32_t* workspace, int32_t rows, int32_t depth, void* stream);
int dew_moe_quantize_rows_fp8(const void* x /* bf16 [rows, K] */, void* codes /* [rows, K] bytes */,
                              uint8_t* scales /* [rows, P] e8m0 */, int32_t rows, int32_t depth, void* stream);
int dew_moe_grouped_gemm_fp8_rows(const void* x_codes, const uint8_t* x_scales, const int32_t* gather,
                                  const int32_t* offsets, const dew_moe_bank* w, const float* bias,
                                  const int32_t* scatter, void* out, int32_t rows, void* stream);

/* gate and up in one launch with the SwiGLU epilogue: hidden[i] = swiglu(x[gather[i]] @ Wg[e], .. @ Wu[e])
 * with the reference's rounding sequence (src/dew/nn/activations.py:267-278): both products rounded to
 * bf16, a = bf16(g * logistic(g)), hidden = bf16(a * u).                                                */
int dew_moe_gateup_swiglu(const void* x, const int32_t* gather, const int32_t* offsets,
                          const dew_moe_bank* gate, const dew_moe_bank* up, void* hidden /* bf16 [rows,F] */,
                          int32_t rows, void* stream);

/* The unfused epilogue alone (src/dew/nn/activations.py:336-356 gated_product('swiglu')).               */
int dew_moe_swiglu(const void* gate, const void* up, void* hidden, int64_t count, void* stream);
/* The same with the gate clamped from above and the up projection both ways by `limit` before their product
 * (`swiglu_clamped`, src/dew/nn/activations.py:327-333: DeepSeek V4's and GLM's experts); limit 0 = none.  */
int dew_moe_swiglu_clamped(const void* gate, const void* up, float limit, void* hidden, int64_t count, void* stream);
/* `gated_product(activation)` for the gates the reference's gated MLPs name besides SwiGLU (src/dew/nn/activations.py:255-265,
 * 336-356): DEW_MOE_GATE_SILU is dew_moe_swiglu_clamped; DEW_MOE_GATE_GELU_TANH is 'geglu', the tanh GELU in its logistic
 * form g * logistic(sqrt(8 / pi) (g + 0.044715 g^3)) (`gelu_tanh`, :57-69: Gemma's experts, src/dew/nn/gemma4_moe.py:84),
 * with the same two roundings and the same optional clamp.                                                           */
enum { DEW_MOE_GATE_SILU = 0, DEW_MOE_GATE_GELU_TANH = 1, DEW_MOE_ACT_RELU2 = 2 /* dew_moe_relu2's own: no gate */ };
int dew_moe_gated_product(const void* gate, const void* up, int32_t activation, float limit, void* hidden, int64_t count, void* stream);
/* dew_moe_gateup_swiglu with that gating as the paired launch's epilogue: hidden = gated_product(activation) of the two
 * products, clamped by `limit` first where that is positive, bit for bit dew_moe_gated_product over the two products of
 * `paired_projections` (src/dew/nn/moe.py:745-770, 1319-1325) without their rows' trip through memory. The groups come
 * as `offsets [E + 1]` or as `group_sizes [E]` (the other NULL). DeepSeek V4's and GLM's clamped experts and Gemma's
 * GeGLU experts take it on every bank format of the bf16-operand launches.                                       */
int dew_moe_gateup_gated(const void* x, const int32_t* gather, const int32_t* offsets /* nullable */,
                         const int32_t* group_sizes /* nullable */, const dew_moe_bank* gate, const dew_moe_bank* up,
                         int32_t activation, float limit, void* hidden, int32_t rows, void* stream);
/* The same paired launch for general NVFP4 banks (DEW_MOE_W_NVFP4: e4m3 block scales with mantissas, `NvFp4`,
 * src/dew/nn/kernels/formats.py:27-137) on f16 operands: `nvfp4_product`'s decode (src/dew/nn/kernels/gemm.py:609-662,
 * formats.py:108-113: code x block scale, exact in bf16) is as exact in f16, where it costs the vector unit one packed
 * conversion and one packed multiply for two codes, half of the bf16 form. dew_moe_rows_f16 brings the rows to f16 under one
 * power-of-two scale a row (halves [rows, depth] f16, scale [rows] e8m0 bytes: x = 2^(scale - 127) halves, the row's largest
 * magnitude in [2^15, 2^16); exact for every element within 2^-29 of it); dew_moe_gateup_gated_f16 is dew_moe_gateup_gated on
 * those rows (gather indexes them and their scales). Each product is the bf16 launch's times a power of two and the sums
 * are fp32, so `hidden` is bit for bit dew_moe_gateup_gated's. No counterpart in the reference, whose decode is XLA's.   */
int dew_moe_rows_f16(const void* x /* bf16 [rows, depth] */, void* halves /* f16 [rows, depth] */, uint8_t* scale /* [rows] */,
                     int32_t rows, int32_t depth, void* stream);
int dew_moe_gateup_gated_f16(const void* x_f16, const uint8_t* x_scale, const int32_t* gather, const int32_t* offsets /* nullable */,
                             const int32_t* group_sizes /* nullable */, const dew_moe_bank* gate, const dew_moe_bank* up,
                             int32_t activation, float limit, void* hidden, int32_t rows, void* stream);
/* Llama 4's input-scaled experts (`scale_inputs`, src/dew/nn/moe.py:1124-1126, 1256-1259: `Llama4TextMoe.forward`): the
 * rows the experts multiply, out[i] = bf16(x[gather[i]] * bf16(weights[slots[i]])) for the sorted positions i < rows
 * (gather = the sort's rows, slots = its order, weights [T*k] the router's). The launches then read `out` without a
 * gather and the combine sums the slots unweighted (weights of one).                                              */
int dew_moe_scale_rows(const void* x /* bf16 [T,D] */, const int32_t* gather, const int32_t* slots, const float* weights,
                       void* out /* bf16 [rows,D] */, int32_t rows, int32_t depth, void* stream);
/* Qwen2-MoE's gate on the shared expert (`shared_gate`, src/dew/nn/moe.py:1469-1475, 1497-1503, under a bf16 compute
 * dtype): out[t, :] = bf16(rows[t, :] * g[t]), g[t] = bf16(logistic(bf16(sum_d x[t, d] * bf16(kernel[d])))), the sum in
 * fp32. rows and out may be the same buffer.                                                                          */
int dew_moe_gate_rows(const void* x /* bf16 [T,D] */, const float* kernel /* [D] */, const void* rows /* bf16 [T,W] */,
                      void* out /* bf16 [T,W] */, int32_t tokens, int32_t depth, int32_t width, void* stream);
/* The same gate where the layer states no compute dtype (src/dew/nn/moe.py:1469-1475, 1497-1503): the gate's Dense(1) then
 * runs in the fp32 of its kernel and the layer's output widens to fp32:
 * out[t, :] = f32(routed[t, :]) + f32(shared[t, :]) * logistic(sum_d x[t, d] * kernel[d]), every operation in fp32.          */
int dew_moe_gate_rows_add_f32(const void* x /* bf16 [T,D] */, const float* kernel /* [D] */, const void* shared /* bf16 [T,W] */,
                              const void* routed /* bf16 [T,W] */, float* out /* [T,W] */, int32_t tokens, int32_t depth,
                              int32_t width, void* stream);

/* Nemotron-H's ungated experts (`activation='relu2'`, src/dew/nn/moe.py:1250-1252, 1319-1322: up_proj, squared ReLU,
 * down_proj): out = bf16(max(x, 0)^2) (`relu2`, src/dew/nn/activations.py:109-111), between two dew_moe_grouped_gemm launches. */
int dew_moe_relu2(const void* x /* bf16 [count] */, void* out /* bf16 [count] */, int64_t count, void* stream);
/* The activation alone: out = bf16(x * logistic(x)), formed in fp32 and rounded once (`silu`, src/dew/nn/activations.py:100-106),
 * which routed value experts pass each chosen projection through (src/dew/nn/value_experts.py:79-82).      */
int dew_moe_silu(const void* x /* bf16 [count] */, void* out /* bf16 [count] */, int64_t count, void* stream);

/* ---- Combine (src/dew/nn/moe.py:1328-1333 `_combine`, :1503 shared add) ----------------------------
 * out[t,:] = bf16( sum_j f32(slots[t,j,:]) * weights[t,j] ), fp32 sum in slot order; with `addend`
 * (the shared expert's output, bf16 [T,D]) out = bf16(f32(out) + f32(addend)).                          */
int dew_moe_combine(const void* slots /* bf16 [T,k,D] */, const float* weights /* [T,k] */,
                    const void* addend /* nullable */, void* out /* bf16 [T,D] */, int32_t tokens,
                    int32_t top_k, int32_t width, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DEW_MOE_HIP_H */
