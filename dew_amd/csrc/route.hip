// Router: scores, (group-limited) selection, top-k and gate weights, one wavefront per token.
// Follows Router.__call__ from the logits on (reference src/dew/nn/moe.py:466-565). Every floating-point
// step is a fixed sequence of IEEE fp32/fp64 operations with contraction off, the same sequence the CPU
// oracle runs, so the chosen experts agree bit for bit.
#include <algorithm>
#include <type_traits>

#include "common.h"

#pragma clang fp contract(off)

namespace dew {

constexpr int kWave = 64;
constexpr int kMaxPerLane = 8;   // experts <= 512
constexpr int kRouteWaves = 4;   // tokens per 256-thread block

// DeepSeek V4's score sqrt(softplus(x)) (src/dew/nn/moe.py:303-313), formed in float64 (softplus as max(x, 0) +
// log1p(exp(-|x|)), the square root IEEE) and rounded once to fp32: the CPU oracle's arithmetic for this score.
__device__ __forceinline__ float sqrt_softplus_f32(float x) {
  const double wide = static_cast<double>(x);
  return static_cast<float>(sqrt(fmax(wide, 0.0) + log1p(exp(-fabs(wide)))));
}

// A score that is a function of its own logit alone (every score function but softmax).
__device__ __forceinline__ float pointwise_score(int score_function, float logit) {
  return score_function == DEW_MOE_SCORE_SQRTSOFTPLUS ? sqrt_softplus_f32(logit) : 1.0f / (1.0f + exp_f32(-logit));
}

// The wavefront's largest value, in every lane: maxima within quads, half rows and rows of 16 lanes by DPP moves (one
// instruction each, no LDS crossbar), then lane 15 of each row into the next row and lane 31 into the upper half, so that
// lane 63 holds the maximum of all 64, which a lane read hands to everyone. (A maximum does not depend on the order it
// is taken in, so this is the butterfly's result; the sums below keep their fixed order.)
__device__ __forceinline__ float wave_max(float v) {
  auto moved = [](float value, auto control, auto rows) {
    const int bits = __builtin_bit_cast(int, value);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(bits, bits, decltype(control)::value, decltype(rows)::value, 0xF, false));
  };
  using std::integral_constant;
  v = fmaxf(v, moved(v, integral_constant<int, 0xB1>{}, integral_constant<int, 0xF>{}));   // quad_perm [1,0,3,2]
  v = fmaxf(v, moved(v, integral_constant<int, 0x4E>{}, integral_constant<int, 0xF>{}));   // quad_perm [2,3,0,1]
  v = fmaxf(v, moved(v, integral_constant<int, 0x141>{}, integral_constant<int, 0xF>{}));  // row_half_mirror
  v = fmaxf(v, moved(v, integral_constant<int, 0x140>{}, integral_constant<int, 0xF>{}));  // row_mirror
  v = fmaxf(v, moved(v, integral_constant<int, 0x142>{}, integral_constant<int, 0xA>{}));  // row_bcast15 into rows 1, 3
  v = fmaxf(v, moved(v, integral_constant<int, 0x143>{}, integral_constant<int, 0xC>{}));  // row_bcast31 into rows 2, 3
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Sum rounded once: fp64 partials per lane, then a butterfly; every lane ends with the same value.
__device__ __forceinline__ float wave_sum_once(double v) {
#pragma unroll
  for (int offset = 32; offset >= 1; offset >>= 1) v = v + __shfl_xor(v, offset, kWave);
  return static_cast<float>(v);
}

struct Best {
  float value;
  int index;
};

__device__ __forceinline__ bool better(float v, int i, const Best& than) {
  return v > than.value || (v == than.value && i < than.index);
}

// The wavefront's best (value, index): the largest value by a butterfly of maxima, then the lowest index among the
// lanes that hold it. Almost always one lane does, found by a ballot and read with one cross-lane move; ties walk
// the ballot's set bits. Half the cross-lane traffic of reducing value and index together.
__device__ __forceinline__ Best wave_best(Best b) {
  const float top = wave_max(b.value);
  unsigned long long holders = __ballot(b.value == top);
  Best best;
  best.value = top;
  best.index = 0x7fffffff;
  while (holders != 0ull) {
    const int lane = __builtin_ctzll(holders);
    best.index = min(best.index, __builtin_amdgcn_readlane(b.index, lane));
    holders &= holders - 1ull;
  }
  return best;
}

struct RouteParams {
  const float* logits;
  const float* bias;
  float* weights;
  int32_t* indices;
  int tokens, experts, top_k, score_function, normalize, expert_groups, groups_per_token;
  int group_by_max;  // a group's score is its best selection (`group_score='max'`), not the sum of its two best
  float scaling;
  float* scores;  // nullable [T, E]: the activated scores, as the router sows them for the balance statistics
  float* log_z;   // nullable [T]: logsumexp of the logits (the z-loss's log partition)
  int bias_in_weights;   // the weights are the chosen scores + bias
  float sum_epsilon, sum_min;
  int fill_excluded;     // an expert outside the kept groups competes at `excluded` rather than -inf
  float excluded;
  float softcap;         // above 0: every logit is read as softcap * tanh(logit / softcap)
  const int32_t* given;    // nullable [T, k]: the experts to use in place of the router's own choice (a replayed record, a hash table's)
  const uint8_t* covered;  // nullable [T]: with `given`, the tokens it covers; the others keep the router's choice
  const float* media_bias; // nullable [E]: the bias a media token's experts are chosen by, in place of `bias`
  const uint8_t* media;    // nullable [T]: the media tokens
  // Block routing (`Router.block_mask`, src/dew/nn/moe.py:566-585): tokens are `rows` x `length`, each in the block of its
  // row that `blocks` numbers (negative: padding, a block of its own); a token chooses among its block's shortlist.
  const int32_t* blocks;   // nullable [T]
  int length;              // tokens a row
  uint32_t* block_keys;    // [rows x (length + 1), E]: a block's best selection for every expert, as ordered keys (0: none yet)
  const uint8_t* allowed;  // [rows x (length + 1), 64]: bit i of byte `lane` set where expert lane + 64 i is on the block's shortlist
  int gather_blocks;       // this launch only gathers the blocks' best selections into block_keys
};

// A float as an unsigned key of the same order (-inf lowest of the non-NaN), never 0.
__device__ __forceinline__ uint32_t ordered_key(float v) {
  const uint32_t bits = __float_as_uint(v);
  return (bits & 0x80000000u) ? ~bits : bits | 0x80000000u;
}

__device__ __forceinline__ float from_ordered_key(uint32_t key) {
  if (key == 0u) return -__builtin_inff();  // no token wrote here
  return __uint_as_float((key & 0x80000000u) ? key & 0x7fffffffu : ~key);
}

// The block a token routes with: its row's blocks are numbered from 0, padding (or an id past the row) is block `length`.
__device__ __forceinline__ size_t block_of(const RouteParams& p, int token) {
  const int id = p.blocks[token];
  return static_cast<size_t>(token / p.length) * (p.length + 1) + ((id < 0 || id > p.length) ? p.length : id);
}

// Laguna's capped gate logit (`capped_logits`, src/dew/nn/precision.py:2086-2092): cap * tanh(logit / cap) in fp32.
__device__ __forceinline__ float capped(float logit, float cap) { return cap > 0.0f ? cap * tanhf(logit / cap) : logit; }

template <int kPerLane>  // experts <= 64 * kPerLane
__global__ __launch_bounds__(kWave* kRouteWaves) void route_kernel(RouteParams p) {
  extern __shared__ float shared[];  // [kRouteWaves][experts] selections, for the group scores
  const int lane = threadIdx.x % kWave;
  const int wave = threadIdx.x / kWave;
  const int token_raw = blockIdx.x * kRouteWaves + wave;
  const bool active = token_raw < p.tokens;
  const int token = active ? token_raw : p.tokens - 1;
  const float* row = p.logits + static_cast<size_t>(token) * p.experts;
  const float ninf = -__builtin_inff();

  float logit[kPerLane], score[kPerLane], select[kPerLane];
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) {
    const int e = lane + kWave * i;
    logit[i] = e < p.experts ? row[e] : ninf;
  }
  if (p.softcap > 0.0f) {  // (a branch of its own: the cap's hyperbolic tangent stays out of the routers that have none)
#pragma unroll
    for (int i = 0; i < kPerLane; ++i)
      if (lane + kWave * i < p.experts) logit[i] = capped(logit[i], p.softcap);
  }

  float top = ninf, denom = 1.0f;
  if (p.score_function == DEW_MOE_SCORE_SOFTMAX) {
    float m = ninf;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) m = fmaxf(m, logit[i]);
    top = wave_max(m);
    double partial = 0.0;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = lane + kWave * i;
      score[i] = e < p.experts ? exp_f32(logit[i] - top) : 0.0f;
      partial = partial + static_cast<double>(score[i]);
    }
    denom = wave_sum_once(partial);
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) score[i] = score[i] / denom;
  } else {
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) score[i] = pointwise_score(p.score_function, logit[i]);
  }

  // What the router sows beside its choices (src/dew/nn/moe.py:474-479): the scores, and the log partition
  // max + log(sum exp(logit - max)) of the logits whatever the score function.
  if (p.scores != nullptr && active) {
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = lane + kWave * i;
      if (e < p.experts) p.scores[static_cast<size_t>(token) * p.experts + e] = score[i];
    }
  }
  if (p.log_z != nullptr) {
    float m = ninf;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) m = fmaxf(m, logit[i]);
    m = wave_max(m);
    double partial = 0.0;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = lane + kWave * i;
      if (e < p.experts) partial = partial + static_cast<double>(exp_f32(logit[i] - m));
    }
    const float total = wave_sum_once(partial);
    if (active && lane == 0) p.log_z[token] = m + logf(total);
  }

  const bool by_media = p.media != nullptr && p.media[token] != 0;  // DeepSeek-V4.1's image-span tokens (one token a wavefront)
#pragma unroll
  for (int i = 0; i < kPerLane; ++i) {
    const int e = lane + kWave * i;
    float s = score[i];
    if (e < p.experts) {
      if (by_media) s = s + p.media_bias[e];
      else if (p.bias != nullptr) s = s + p.bias[e];
    }
    // A NaN selection (a NaN in the bias or the logits) is never preferred: it competes as -inf, so every round still
    // finds an expert in range (no comparison with NaN holds, and a round without a candidate would name no expert).
    select[i] = (e < p.experts && s == s) ? s : ninf;
  }

  if (p.blocks != nullptr) {  // (a block router has no expert groups: no barrier lies ahead of the early return)
    const size_t block = block_of(p, token);
    if (p.gather_blocks) {
      if (active) {
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) {
          const int e = lane + kWave * i;
          if (e < p.experts) atomicMax(p.block_keys + block * p.experts + e, ordered_key(select[i]));
        }
      }
      return;
    }
    const unsigned shortlist = p.allowed[block * kWave + lane];
#pragma unroll
    for (int i = 0; i < kPerLane; ++i)
      if (!((shortlist >> i) & 1u)) select[i] = ninf;
  }

  if (p.expert_groups > 1) {
    float* mine = shared + wave * p.experts;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = lane + kWave * i;
      if (e < p.experts) mine[e] = select[i];
    }
    __syncthreads();
    const int per_group = p.experts / p.expert_groups;
    // lane g scores group g: the sum of its two best selections
    float group_score = ninf;
    if (lane < p.expert_groups) {
      float first = ninf, second = ninf;
      for (int j = 0; j < per_group; ++j) {
        const float v = mine[lane * per_group + j];
        if (v > first) {
          second = first;
          first = v;
        } else if (v > second) {
          second = v;
        }
      }
      group_score = p.group_by_max ? first : first + second;
    }
    unsigned long long kept = 0ull;
    bool taken = false;
    for (int round = 0; round < p.groups_per_token; ++round) {
      Best b;
      b.value = ninf;
      b.index = 0x7fffffff;
      if (lane < p.expert_groups && !taken) {
        b.value = group_score;
        b.index = lane;
      }
      b = wave_best(b);
      kept |= 1ull << b.index;
      if (b.index == lane) taken = true;
    }
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = lane + kWave * i;
      if (e < p.experts && !((kept >> (e / per_group)) & 1ull)) select[i] = p.fill_excluded ? p.excluded : ninf;
    }
  }

  // A token whose experts are given takes them as they come; the wavefront is one token, so the branch is uniform. A given
  // id outside [0, experts) (a dropped slot's sentinel in a replayed record) is written back as it came, with weight zero
  // and no part in the other slots' normalization: the reference passes such ids through (`chosen_experts`,
  // src/dew/nn/moe.py:202-224) and its sort drops the slot. Its reads below go to the nearest expert, to stay in range.
  const bool replayed = p.given != nullptr && (p.covered == nullptr || p.covered[token] != 0);
  // top-k: k rounds of a wave-wide argmax, ties to the lower index
  unsigned taken_mask = 0u;
  int my_choice = 0, given_id = 0;
  bool in_range = true;
  if (replayed && lane < p.top_k) {
    given_id = p.given[static_cast<size_t>(token) * p.top_k + lane];
    in_range = given_id >= 0 && given_id < p.experts;
    my_choice = min(max(given_id, 0), p.experts - 1);
  }
  for (int round = 0; round < (replayed ? 0 : p.top_k); ++round) {
    Best b;
    b.value = ninf;
    b.index = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
      const int e = lane + kWave * i;
      if (e < p.experts && !((taken_mask >> i) & 1u) && better(select[i], e, b)) {
        b.value = select[i];
        b.index = e;
      }
    }
    b = wave_best(b);
    if ((b.index % kWave) == lane) taken_mask |= 1u << (b.index / kWave);
    if (lane == round) my_choice = min(b.index, p.experts - 1);
  }

  // gate weights: lane j < k owns the j-th choice
  const bool owner = lane < p.top_k && in_range;
  float chosen_logit = owner ? row[my_choice] : ninf;
  if (p.softcap > 0.0f && owner) chosen_logit = capped(chosen_logit, p.softcap);
  float weight = 0.0f;
  if (p.score_function == DEW_MOE_SCORE_SOFTMAX && p.normalize && !p.bias_in_weights && !(p.sum_min != 0.0f)) {
    const float m = wave_max(chosen_logit);
    const float shifted = owner ? exp_f32(chosen_logit - m) : 0.0f;
    const float total = wave_sum_once(static_cast<double>(shifted));
    weight = shifted / total;
  } else {
    if (owner) {
      weight = p.score_function == DEW_MOE_SCORE_SOFTMAX ? exp_f32(chosen_logit - top) / denom
                                                         : pointwise_score(p.score_function, chosen_logit);
      if (p.bias_in_weights) weight = weight + p.bias[my_choice];
    }
    if (p.normalize) {
      float total = __shfl(weight, 0, kWave);
      for (int j = 1; j < p.top_k; ++j) total = total + __shfl(weight, j, kWave);
      total = total + p.sum_epsilon;
      if (p.sum_min != 0.0f) total = fmaxf(total, p.sum_min);
      weight = weight / total;
    }
  }
  weight = weight * p.scaling;
  if (active && lane < p.top_k) {
    p.weights[static_cast<size_t>(token) * p.top_k + lane] = in_range ? weight : 0.0f;
    p.indices[static_cast<size_t>(token) * p.top_k + lane] = replayed ? given_id : my_choice;
  }
}

// Each block's shortlist: the `count` best of its best selections (ties to the lower index), one wavefront a block.
__global__ __launch_bounds__(kWave* kRouteWaves) void block_shortlist_kernel(const uint32_t* __restrict__ keys, uint8_t* __restrict__ allowed,
                                                                             int blocks, int experts, int count) {
  const int lane = threadIdx.x % kWave;
  const int block = blockIdx.x * kRouteWaves + threadIdx.x / kWave;
  if (block >= blocks) return;
  float best[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int e = lane + kWave * i;
    best[i] = e < experts ? from_ordered_key(keys[static_cast<size_t>(block) * experts + e]) : -__builtin_inff();
  }
  unsigned taken = 0u;
  for (int round = 0; round < count; ++round) {
    Best b;
    b.value = -__builtin_inff();
    b.index = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int e = lane + kWave * i;
      if (e < experts && !((taken >> i) & 1u) && better(best[i], e, b)) {
        b.value = best[i];
        b.index = e;
      }
    }
    b = wave_best(b);
    if ((b.index % kWave) == lane) taken |= 1u << (b.index / kWave);
  }
  allowed[static_cast<size_t>(block) * kWave + lane] = static_cast<uint8_t>(taken);
}

__global__ __launch_bounds__(256) void clear_words_kernel(uint32_t* __restrict__ words, size_t count) {
  for (size_t i = blockIdx.x * 256ull + threadIdx.x; i < count; i += static_cast<size_t>(gridDim.x) * 256) words[i] = 0u;
}

}  // namespace dew

extern "C" int dew_moe_route(const float* logits, const float* bias, int32_t tokens, int32_t experts,
                             int32_t top_k, int32_t score_function, int32_t normalize, float scaling,
                             int32_t expert_groups, int32_t groups_per_token, float* weights,
                             int32_t* indices, void* stream) {
  return dew_moe_route_sown(logits, bias, tokens, experts, top_k, score_function, normalize, scaling, expert_groups,
                            groups_per_token, weights, indices, nullptr, nullptr, stream);
}

extern "C" int dew_moe_route_sown(const float* logits, const float* bias, int32_t tokens, int32_t experts,
                                  int32_t top_k, int32_t score_function, int32_t normalize, float scaling,
                                  int32_t expert_groups, int32_t groups_per_token, float* weights,
                                  int32_t* indices, float* scores, float* log_z, void* stream) {
  const dew_moe_router router{experts, top_k, score_function, normalize, scaling, expert_groups, groups_per_token,
                              DEW_MOE_GROUP_TOP2, 0, DEW_MOE_WEIGHT_SUM_EPSILON, 0.0f, 0, 0.0f, 0.0f};
  return dew_moe_route_with(&router, logits, bias, tokens, weights, indices, scores, log_z, stream);
}

extern "C" int dew_moe_route_with(const dew_moe_router* router, const float* logits, const float* bias, int32_t tokens,
                                  float* weights, int32_t* indices, float* scores, float* log_z, void* stream) {
  return dew_moe_route_call(router, logits, bias, nullptr, nullptr, nullptr, nullptr, tokens, weights, indices, scores, log_z, stream);
}

namespace dew {
struct BlockRouting {
  const int32_t* blocks = nullptr;
  int length = 0;
  uint32_t* keys = nullptr;
  const uint8_t* allowed = nullptr;
  int gather = 0;
};
static int route_launch(const dew_moe_router* router, const float* logits, const float* bias, const float* media_bias,
                        const uint8_t* media, const int32_t* given, const uint8_t* covered, const BlockRouting& by_block,
                        int32_t tokens, float* weights, int32_t* indices, float* scores, float* log_z, void* stream);
}  // namespace dew

extern "C" int dew_moe_route_call(const dew_moe_router* router, const float* logits, const float* bias,
                                  const float* media_bias, const uint8_t* media, const int32_t* given,
                                  const uint8_t* covered, int32_t tokens, float* weights, int32_t* indices, float* scores,
                                  float* log_z, void* stream) {
  return dew::route_launch(router, logits, bias, media_bias, media, given, covered, dew::BlockRouting{}, tokens, weights, indices,
                           scores, log_z, stream);
}

int dew::route_launch(const dew_moe_router* router, const float* logits, const float* bias, const float* media_bias,
                             const uint8_t* media, const int32_t* given, const uint8_t* covered, const BlockRouting& by_block,
                             int32_t tokens, float* weights, int32_t* indices, float* scores, float* log_z, void* stream) {
  DEW_REQUIRE(given || !covered, "dew_moe_route: a coverage without the experts it covers");
  DEW_REQUIRE((media == nullptr) == (media_bias == nullptr), "dew_moe_route: the media tokens and the bias that chooses for them come together");
  DEW_REQUIRE(router, "dew_moe_route: the router's description must not be null");
  const int experts = router->experts, top_k = router->top_k, score_function = router->score_function;
  const int expert_groups = router->expert_groups, groups_per_token = router->groups_per_token;
  DEW_REQUIRE(tokens >= 0 && experts >= 1, "dew_moe_route: tokens %d experts %d", tokens, experts);
  DEW_REQUIRE(tokens == 0 || (logits && weights && indices), "dew_moe_route: logits, weights and indices must not be null");
  DEW_REQUIRE(experts <= kWave * kMaxPerLane, "dew_moe_route: at most %d experts, got %d", kWave * kMaxPerLane,
              experts);
  DEW_REQUIRE(top_k >= 1 && top_k <= experts && top_k <= kWave, "dew_moe_route: top_k %d of %d experts (at most %d)",
              top_k, experts, kWave);
  DEW_REQUIRE(score_function == DEW_MOE_SCORE_SOFTMAX || score_function == DEW_MOE_SCORE_SIGMOID || score_function == DEW_MOE_SCORE_SQRTSOFTPLUS,
              "dew_moe_route: score_function %d is none of softmax (0), sigmoid (1), sqrtsoftplus (2)", score_function);
  DEW_REQUIRE(router->group_score == DEW_MOE_GROUP_TOP2 || router->group_score == DEW_MOE_GROUP_MAX,
              "dew_moe_route: group_score %d is neither top2 (0) nor max (1)", router->group_score);
  DEW_REQUIRE(expert_groups >= 1 && expert_groups <= kWave && experts % expert_groups == 0,
              "dew_moe_route: %d experts do not split into %d groups (at most %d)", experts, expert_groups, kWave);
  if (expert_groups > 1) {
    DEW_REQUIRE(groups_per_token >= 1 && groups_per_token <= expert_groups,
                "dew_moe_route: groups_per_token %d of %d groups", groups_per_token, expert_groups);
    DEW_REQUIRE(experts / expert_groups >= 2 || router->group_score == DEW_MOE_GROUP_MAX,
                "dew_moe_route: a group's score sums its two best experts, got %d a group", experts / expert_groups);
    DEW_REQUIRE(top_k <= groups_per_token * (experts / expert_groups),
                "dew_moe_route: top_k %d exceeds the %d experts of the kept groups", top_k,
                groups_per_token * (experts / expert_groups));
  }
  DEW_REQUIRE(!router->bias_in_weights || bias, "dew_moe_route: bias_in_weights gates on the balancing bias, which is null");
  DEW_REQUIRE(router->weight_sum_epsilon >= 0.0f && router->weight_sum_min >= 0.0f,
              "dew_moe_route: weight_sum_epsilon %g and weight_sum_min %g bound a sum from below: neither is negative",
              static_cast<double>(router->weight_sum_epsilon), static_cast<double>(router->weight_sum_min));
  DEW_REQUIRE(router->logit_softcap >= 0.0f, "dew_moe_route: logit_softcap %g is a positive cap, or 0 for none",
              static_cast<double>(router->logit_softcap));
  if (tokens == 0) return DEW_MOE_OK;
  RouteParams p{logits, bias, weights, indices, tokens, experts, top_k, score_function, router->normalize ? 1 : 0,
                expert_groups, groups_per_token, router->group_score == DEW_MOE_GROUP_MAX ? 1 : 0, router->scaling, scores, log_z,
                router->bias_in_weights ? 1 : 0, router->weight_sum_epsilon, router->weight_sum_min,
                router->fill_excluded ? 1 : 0, router->excluded_group_score, router->logit_softcap, given, covered, media_bias, media,
                by_block.blocks, by_block.length, by_block.keys, by_block.allowed, by_block.gather};
  const int blocks = (tokens + kRouteWaves - 1) / kRouteWaves;
  const size_t shared = expert_groups > 1 ? sizeof(float) * kRouteWaves * experts : 0;
  const dim3 grid(blocks), block(kWave * kRouteWaves);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (experts <= 64) {
    hipLaunchKernelGGL(route_kernel<1>, grid, block, shared, s, p);
  } else if (experts <= 128) {
    hipLaunchKernelGGL(route_kernel<2>, grid, block, shared, s, p);
  } else if (experts <= 256) {
    hipLaunchKernelGGL(route_kernel<4>, grid, block, shared, s, p);
  } else {
    hipLaunchKernelGGL(route_kernel<kMaxPerLane>, grid, block, shared, s, p);
  }
  return launched("route_kernel");
}

extern "C" size_t dew_moe_route_blocks_workspace_bytes(int32_t rows, int32_t length, int32_t experts) {
  if (rows <= 0 || length <= 0 || experts <= 0) return 0;
  const size_t blocks = static_cast<size_t>(rows) * (static_cast<size_t>(length) + 1);
  return blocks * experts * sizeof(uint32_t) + blocks * dew::kWave;
}

extern "C" int dew_moe_route_blocks(const dew_moe_router* router, const float* logits, const float* bias,
                                    const int32_t* blocks, int32_t rows, int32_t length, int32_t block_experts,
                                    void* workspace, size_t workspace_bytes, float* weights, int32_t* indices, float* scores,
                                    float* log_z, void* stream) {
  using namespace dew;
  DEW_REQUIRE(router, "dew_moe_route_blocks: the router's description must not be null");
  DEW_REQUIRE(rows >= 0 && length >= 1 && static_cast<long long>(rows) * length <= 0x7fffffffLL,
              "dew_moe_route_blocks: %d rows of %d tokens", rows, length);
  DEW_REQUIRE(router->expert_groups == 1, "dew_moe_route_blocks: block routing limits a token to its block's experts, so it has no expert groups");
  DEW_REQUIRE(block_experts >= router->top_k && block_experts <= router->experts,
              "dew_moe_route_blocks: block_experts %d must hold the top_k of %d and at most the %d experts", block_experts,
              router->top_k, router->experts);
  if (rows == 0) return DEW_MOE_OK;
  DEW_REQUIRE(blocks, "dew_moe_route_blocks: the tokens' blocks must not be null");
  const size_t needed = dew_moe_route_blocks_workspace_bytes(rows, length, router->experts);
  DEW_REQUIRE(workspace && workspace_bytes >= needed && reinterpret_cast<uintptr_t>(workspace) % 4 == 0,
              "dew_moe_route_blocks: the workspace holds %zu bytes of the %zu needed (dew_moe_route_blocks_workspace_bytes), 4-byte aligned",
              workspace ? workspace_bytes : size_t{0}, needed);
  const int tokens = rows * length;
  const size_t segments = static_cast<size_t>(rows) * (static_cast<size_t>(length) + 1);
  const size_t words = segments * router->experts;
  uint32_t* keys = static_cast<uint32_t*>(workspace);
  uint8_t* allowed = reinterpret_cast<uint8_t*>(keys + words);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // (a kernel, not a memset: a caller may capture these launches in a graph)
  hipLaunchKernelGGL(clear_words_kernel, dim3(static_cast<unsigned>(std::min<size_t>((words + 255) / 256, 4096))), dim3(256), 0, s, keys, words);
  BlockRouting by_block;
  by_block.blocks = blocks, by_block.length = length, by_block.keys = keys, by_block.allowed = allowed, by_block.gather = 1;
  int status = route_launch(router, logits, bias, nullptr, nullptr, nullptr, nullptr, by_block, tokens, weights, indices, nullptr, nullptr, stream);
  if (status != DEW_MOE_OK) return status;
  hipLaunchKernelGGL(block_shortlist_kernel, dim3(static_cast<unsigned>((segments + kRouteWaves - 1) / kRouteWaves)), dim3(kWave * kRouteWaves),
                     0, s, keys, allowed, static_cast<int>(segments), router->experts, block_experts);
  by_block.gather = 0;
  return route_launch(router, logits, bias, nullptr, nullptr, nullptr, nullptr, by_block, tokens, weights, indices, scores, log_z, stream);
}

namespace dew {

// The aux-loss-free balancing step on the selection bias (src/dew/nn/moe.py:271-300 `load_balance_update`, applied
// as src/dew/objectives/routing.py:342-345): an expert that took more slots than the average loses `rate`, one that
// took fewer gains it, one exactly at the floor of the average gains it only if the average has a remainder.
__global__ __launch_bounds__(256) void balance_bias_kernel(const int32_t* __restrict__ counts, float* __restrict__ bias,
                                                           float rate, int experts) {
  __shared__ long long partial[256];
  long long sum = 0;
  for (int e = threadIdx.x; e < experts; e += 256) sum += counts[e];
  partial[threadIdx.x] = sum;
  __syncthreads();
  for (int half = 128; half >= 1; half >>= 1) {
    if (threadIdx.x < half) partial[threadIdx.x] += partial[threadIdx.x + half];
    __syncthreads();
  }
  const long long total = partial[0];
  const long long average = total / experts, remainder = total % experts;
  for (int e = threadIdx.x; e < experts; e += 256) {
    const long long count = counts[e];
    const float direction = count > average ? -1.0f : (count < average || remainder > 0) ? 1.0f : 0.0f;
    bias[e] = bias[e] + rate * direction;
  }
}

}  // namespace dew

extern "C" int dew_moe_balance_bias(const int32_t* counts, float* bias, float rate, int32_t experts, void* stream) {
  using namespace dew;
  DEW_REQUIRE(experts >= 1, "dew_moe_balance_bias: experts %d", experts);
  DEW_REQUIRE(counts && bias, "dew_moe_balance_bias: counts and bias must not be null");
  hipLaunchKernelGGL(balance_bias_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream), counts, bias, rate, experts);
  return launched("balance_bias_kernel");
}
