// Dispatch bookkeeping: the stable counting sort of routed slots by expert id
// (reference src/dew/nn/moe.py:1101-1128 `_sorted_locally`: argsort(experts), bincount, order // k).
//
// Three stream-ordered launches, no global atomics, so the result is deterministic:
//   count   each 2048-slot block builds an LDS histogram of its slots (one sub-histogram per wavefront)
//   scan    one block turns the per-block counts into sizes, offsets and each block's base per expert
//   scatter each wavefront ranks its 64 slots among themselves with ballots (match-any over the id's bits),
//           adds the running count of earlier slots, and writes order[] / rows[]
// Slots whose id is >= experts (a dropped slot's sentinel) sort last, in slot order, outside every group.
#include <mutex>

#include "common.h"

namespace dew {

constexpr int kPermuteThreads = 256;
constexpr int kPermuteWaves = kPermuteThreads / 64;
constexpr int kSlotsPerBlock = 2048;
constexpr int kSlotsPerWave = kSlotsPerBlock / kPermuteWaves;
constexpr int kMaxExperts = 1024;  // buckets = experts + 1 (the sentinel's) <= 1025 handled by loops

struct PermuteParams {
  const int32_t* ids;  // [slots]
  int32_t* sizes;      // [experts]
  int32_t* offsets;    // [experts + 1]
  int32_t* order;      // [slots]
  int32_t* rows;       // [slots]
  int32_t* counts;     // workspace [blocks][buckets]
  int32_t* bases;      // workspace [blocks][buckets]
  // `slots` sorted positions: the `routed` = tokens * top_k slots of `ids`, then `slots - routed` rows that every token
  // sends to one always-on (shared) expert, which sorts as group `experts`. `groups` = the groups written (experts, or
  // experts + 1 with a shared one); bucket `groups` collects the dropped slots (an id outside [0, experts)), last.
  int slots, routed, experts, groups, top_k, blocks, buckets;
};

__device__ __forceinline__ int bucket_of(const PermuteParams& p, int slot) {
  if (slot >= p.routed) return p.experts;  // a shared expert's row
  const int id = p.ids[slot];
  return (id < 0 || id >= p.experts) ? p.groups : id;
}

// The row of the activations a slot reads: its token, or for a shared expert's row the token it is.
__device__ __forceinline__ int row_of(const PermuteParams& p, int slot) {
  return slot < p.routed ? slot / p.top_k : slot - p.routed;
}

__global__ __launch_bounds__(kPermuteThreads) void permute_count_kernel(PermuteParams p) {
  extern __shared__ int32_t hist[];  // [buckets]
  for (int b = threadIdx.x; b < p.buckets; b += kPermuteThreads) hist[b] = 0;
  __syncthreads();
  const int begin = blockIdx.x * kSlotsPerBlock;
  const int end = min(begin + kSlotsPerBlock, p.slots);
  for (int slot = begin + threadIdx.x; slot < end; slot += kPermuteThreads)
    atomicAdd(&hist[bucket_of(p, slot)], 1);
  __syncthreads();
  for (int b = threadIdx.x; b < p.buckets; b += kPermuteThreads)
    p.counts[static_cast<size_t>(blockIdx.x) * p.buckets + b] = hist[b];
}

// One block: totals per bucket, exclusive scan over buckets, then each block's base per bucket.
__global__ __launch_bounds__(kPermuteThreads) void permute_scan_kernel(PermuteParams p) {
  extern __shared__ int32_t totals[];  // [buckets + 1]
  __shared__ int32_t wave_sums[kPermuteThreads / 64];
  for (int b = threadIdx.x; b < p.buckets; b += kPermuteThreads) {
    int sum = 0;
#pragma unroll 8
    for (int blk = 0; blk < p.blocks; ++blk) sum += p.counts[static_cast<size_t>(blk) * p.buckets + b];
    totals[b] = sum;
  }
  __syncthreads();
  // Exclusive scan over the buckets (integer sums: any order is exact): each thread owns a run of consecutive buckets,
  // the runs' sums are scanned across the wavefront by shuffles and across the wavefronts through LDS.
  const int per = (p.buckets + kPermuteThreads - 1) / kPermuteThreads;
  const int first = min(static_cast<int>(threadIdx.x) * per, p.buckets), last = min(first + per, p.buckets);
  int mine = 0;
  for (int b = first; b < last; ++b) mine += totals[b];
  int through = mine;  // inclusive scan of the runs' sums within the wavefront
  const int lane = threadIdx.x % 64;
#pragma unroll
  for (int offset = 1; offset < 64; offset <<= 1) {
    const int below = __shfl_up(through, offset, 64);
    if (lane >= offset) through += below;
  }
  if (lane == 63) wave_sums[threadIdx.x / 64] = through;
  __syncthreads();
  int running = through - mine;
  for (int w = 0; w < static_cast<int>(threadIdx.x) / 64; ++w) running += wave_sums[w];
  for (int b = first; b < last; ++b) {
    const int size = totals[b];
    totals[b] = running;
    running += size;
  }
  if (threadIdx.x == kPermuteThreads - 1) totals[p.buckets] = running;  // the last thread's run ends the buckets (or is empty behind them)
  __syncthreads();
  for (int b = threadIdx.x; b < p.buckets; b += kPermuteThreads) {
    const int start = totals[b];
    if (b < p.groups) {
      p.sizes[b] = totals[b + 1] - start;
      p.offsets[b] = start;
    } else {
      p.offsets[p.groups] = start;  // slots routed to a real expert
    }
    int next = start;
#pragma unroll 8
    for (int blk = 0; blk < p.blocks; ++blk) {
      const size_t at = static_cast<size_t>(blk) * p.buckets + b;
      const int count = p.counts[at];
      p.bases[at] = next;
      next += count;
    }
  }
}

__global__ __launch_bounds__(kPermuteThreads) void permute_scatter_kernel(PermuteParams p) {
  extern __shared__ int32_t running[];  // [kPermuteWaves][buckets]: next free position per wave and bucket
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  const int block_begin = blockIdx.x * kSlotsPerBlock;
  // pass 1: each wave counts its own contiguous 512 slots
  for (int i = threadIdx.x; i < kPermuteWaves * p.buckets; i += kPermuteThreads) running[i] = 0;
  __syncthreads();
  int32_t* mine = running + wave * p.buckets;
  const int wave_begin = block_begin + wave * kSlotsPerWave;
  for (int round = 0; round < kSlotsPerWave / 64; ++round) {
    const int slot = wave_begin + round * 64 + lane;
    if (slot < p.slots) atomicAdd(&mine[bucket_of(p, slot)], 1);
  }
  __syncthreads();
  // turn the per-wave counts into each wave's first position: block base + earlier waves' counts
  for (int b = threadIdx.x; b < p.buckets; b += kPermuteThreads) {
    int next = p.bases[static_cast<size_t>(blockIdx.x) * p.buckets + b];
    for (int w = 0; w < kPermuteWaves; ++w) {
      const int count = running[w * p.buckets + b];
      running[w * p.buckets + b] = next;
      next += count;
    }
  }
  __syncthreads();
  // pass 2: rank within the round by ballots, then advance the wave's running positions
  int bits = 1;
  while ((1 << bits) < p.buckets) ++bits;
  for (int round = 0; round < kSlotsPerWave / 64; ++round) {
    const int slot = wave_begin + round * 64 + lane;
    const bool valid = slot < p.slots;
    const int bucket = valid ? bucket_of(p, slot) : p.buckets;  // invalid lanes match nobody real
    unsigned long long same = __ballot(valid);
    for (int bit = 0; bit < bits; ++bit) {
      const bool set = (bucket >> bit) & 1;
      const unsigned long long vote = __ballot(set);
      same &= set ? vote : ~vote;
    }
    const unsigned long long below = same & ((1ull << lane) - 1ull);
    const int rank = __popcll(below);
    const int count = __popcll(same);
    int position = 0;
    if (valid) position = mine[bucket] + rank;
    __syncthreads();
    if (valid && rank == count - 1) mine[bucket] = position + 1;
    __syncthreads();
    if (valid) {
      p.order[position] = slot;
      p.rows[position] = row_of(p, slot);
    }
  }
}

// All of the above in one launch for at most kSmallSlots slots (a decode step, a small prefill): one block
// counts, scans and scatters, each wavefront a contiguous run of the slots, with the LDS histogram as the only
// intermediate.
// Measured under graph replay, sixteen wavefronts: 2048 slots 5.1 to 6.8 us (four wavefronts: 7.9 to 10.0), 4096 slots
// 7.5 us against 11.4 us for the three launches, 8192 slots the same either way.
constexpr int kSmallSlots = 4096;      // beyond this three launches over many blocks are as fast or faster
constexpr int kSmallThreads = 1024;    // sixteen wavefronts, where their counters fit the LDS a launch may take unasked
constexpr int kNarrowSmallSlots = 2048;  // the four-wavefront form's reach, for more buckets than that
template <int THREADS>
__global__ __launch_bounds__(THREADS) void permute_small_kernel(PermuteParams p) {
  constexpr int kWaves = THREADS / 64;
  extern __shared__ int32_t running[];  // [kWaves][buckets] then [buckets + 1] totals
  int32_t* totals = running + kWaves * p.buckets;
  const int lane = threadIdx.x % 64;
  const int wave = threadIdx.x / 64;
  for (int i = threadIdx.x; i < kWaves * p.buckets; i += THREADS) running[i] = 0;
  __syncthreads();
  int32_t* mine = running + wave * p.buckets;
  const int segment = ((p.slots + THREADS - 1) / THREADS) * 64;  // contiguous slots per wavefront
  const int rounds = segment / 64;
  const int wave_begin = wave * segment;
  // a lane's buckets stay in registers between the count and the scatter (one round trip to the indices, not two)
  constexpr int kMaxRounds = (THREADS == kSmallThreads ? kSmallSlots : kNarrowSmallSlots) / THREADS;
  int kept[kMaxRounds];
#pragma unroll
  for (int round = 0; round < kMaxRounds; ++round) {
    const int slot = wave_begin + round * 64 + lane;
    kept[round] = (round < rounds && slot < p.slots) ? bucket_of(p, slot) : p.buckets;
  }
#pragma unroll
  for (int round = 0; round < kMaxRounds; ++round)
    if (kept[round] < p.buckets) atomicAdd(&mine[kept[round]], 1);
  __syncthreads();
  for (int b = threadIdx.x; b < p.buckets; b += THREADS) {
    int sum = 0;
    for (int w = 0; w < kWaves; ++w) sum += running[w * p.buckets + b];
    totals[b] = sum;
  }
  __syncthreads();
  if (threadIdx.x < 64) {  // exclusive scan of the bucket totals by one wavefront, 64 buckets a round
    int carried = 0;
    for (int base = 0; base < p.buckets; base += 64) {
      const int b = base + lane;
      const int size = b < p.buckets ? totals[b] : 0;
      int inclusive = size;
#pragma unroll
      for (int offset = 1; offset < 64; offset <<= 1) {
        const int other = __shfl_up(inclusive, offset, 64);
        if (lane >= offset) inclusive += other;
      }
      if (b < p.buckets) totals[b] = carried + inclusive - size;
      carried += __shfl(inclusive, 63, 64);
    }
    if (lane == 0) totals[p.buckets] = carried;
  }
  __syncthreads();
  for (int b = threadIdx.x; b < p.buckets; b += THREADS) {
    const int start = totals[b];
    if (b < p.groups) {
      p.sizes[b] = totals[b + 1] - start;
      p.offsets[b] = start;
    } else {
      p.offsets[p.groups] = start;
    }
    int next = start;
    for (int w = 0; w < kWaves; ++w) {
      const int count = running[w * p.buckets + b];
      running[w * p.buckets + b] = next;
      next += count;
    }
  }
  __syncthreads();
  int bits = 1;
  while ((1 << bits) < p.buckets) ++bits;
#pragma unroll
  for (int round = 0; round < kMaxRounds; ++round) {
    if (round >= rounds) continue;  // (the same for the whole block)
    const int slot = wave_begin + round * 64 + lane;
    const int bucket = kept[round];
    const bool valid = bucket < p.buckets;
    unsigned long long same = __ballot(valid);
    for (int bit = 0; bit < bits; ++bit) {
      const bool set = (bucket >> bit) & 1;
      const unsigned long long vote = __ballot(set);
      same &= set ? vote : ~vote;
    }
    const int rank = __popcll(same & ((1ull << lane) - 1ull));
    const int count = __popcll(same);
    int position = 0;
    if (valid) position = mine[bucket] + rank;
    // The running positions are the wavefront's own (no other wavefront touches them), so no block barrier is needed,
    // only an order between this wavefront's lanes: every lane's read above before the one lane's write below, and that
    // write before the next round's reads. The wavefront-scope fences state that order to the compiler and the memory
    // model (they cost no instruction: a wavefront's LDS operations are issued and served in order).
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (valid && rank == count - 1) mine[bucket] = position + 1;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (valid) {
      p.order[position] = slot;
      p.rows[position] = row_of(p, slot);
    }
  }
}

}  // namespace dew

extern "C" size_t dew_moe_permute_workspace_bytes(int32_t slots, int32_t experts) {
  if (slots <= 0 || experts <= 0) return 256;
  const size_t blocks = (static_cast<size_t>(slots) + dew::kSlotsPerBlock - 1) / dew::kSlotsPerBlock;
  return 2 * blocks * (static_cast<size_t>(experts) + 1) * sizeof(int32_t) + 256;
}

namespace dew {

// Capacity dropping (`capacity_positions`, src/dew/nn/moe.py:832-855, applied at :914-919): a block a sequence. Each of a
// sequence's `slots` = length * top_k slots queues at its expert in slot order; a slot whose place in the queue is
// `capacity` or later is dropped: its id becomes `experts`, the sentinel that sorts last and outside every group.
// The place is the slot's rank among its sequence's slots of the same expert: the single block's counting sort above,
// without the scatter.
__global__ __launch_bounds__(kPermuteThreads) void capacity_admit_kernel(const int32_t* __restrict__ ids, int32_t* __restrict__ admitted,
                                                                         int slots, int experts, int capacity) {
  extern __shared__ int32_t running[];  // [kPermuteWaves][buckets]
  const int buckets = experts + 1;
  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int32_t* mine_ids = ids + static_cast<size_t>(blockIdx.x) * slots;
  int32_t* out = admitted + static_cast<size_t>(blockIdx.x) * slots;
  for (int i = threadIdx.x; i < kPermuteWaves * buckets; i += kPermuteThreads) running[i] = 0;
  __syncthreads();
  int32_t* mine = running + wave * buckets;
  const int segment = ((slots + kPermuteThreads - 1) / kPermuteThreads) * 64;  // contiguous slots per wavefront
  const int rounds = segment / 64, wave_begin = wave * segment;
  auto bucket_at = [&](int slot) {
    const int id = mine_ids[slot];
    return (id < 0 || id >= experts) ? experts : id;
  };
  for (int round = 0; round < rounds; ++round) {
    const int slot = wave_begin + round * 64 + lane;
    if (slot < slots) atomicAdd(&mine[bucket_at(slot)], 1);
  }
  __syncthreads();
  for (int b = threadIdx.x; b < buckets; b += kPermuteThreads) {  // each wavefront's first place in every queue
    int next = 0;
    for (int w = 0; w < kPermuteWaves; ++w) {
      const int count = running[w * buckets + b];
      running[w * buckets + b] = next;
      next += count;
    }
  }
  __syncthreads();
  int bits = 1;
  while ((1 << bits) < buckets) ++bits;
  for (int round = 0; round < rounds; ++round) {
    const int slot = wave_begin + round * 64 + lane;
    const bool valid = slot < slots;
    const int bucket = valid ? bucket_at(slot) : buckets;
    unsigned long long same = __ballot(valid);
    for (int bit = 0; bit < bits; ++bit) {
      const bool set = (bucket >> bit) & 1;
      const unsigned long long vote = __ballot(set);
      same &= set ? vote : ~vote;
    }
    const int rank = __popcll(same & ((1ull << lane) - 1ull));
    const int count = __popcll(same);
    int place = 0;
    if (valid) place = mine[bucket] + rank;
    __syncthreads();
    if (valid && rank == count - 1) mine[bucket] = place + 1;
    __syncthreads();
    if (valid) out[slot] = (bucket < experts && place < capacity) ? bucket : experts;
  }
}

// The sort's launches, given where the per-block counts and bases live (the caller's workspace or the library's own
// scratch array): `counts` holds 2 * blocks * buckets int32, 256-byte aligned.
static int permute_launches(const int32_t* indices, int32_t tokens, int32_t top_k, int32_t experts, int32_t shared_rows,
                            int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows, int32_t* counts, hipStream_t s) {
  const int slots = tokens * top_k + shared_rows;
  PermuteParams p;
  p.ids = indices;
  p.sizes = sizes;
  p.offsets = offsets;
  p.order = order;
  p.rows = rows;
  p.slots = slots;
  p.routed = tokens * top_k;
  p.experts = experts;
  p.groups = experts + (shared_rows > 0 ? 1 : 0);
  p.top_k = top_k;
  p.buckets = p.groups + 1;
  p.blocks = (slots + kSlotsPerBlock - 1) / kSlotsPerBlock;
  p.counts = counts;
  p.bases = p.counts + static_cast<size_t>(p.blocks) * p.buckets;
  // one block does it all faster than three launches
  const size_t wide_lds = sizeof(int32_t) * ((kSmallThreads / 64 + 1) * static_cast<size_t>(p.buckets) + 1);
  if (slots <= kSmallSlots && wide_lds <= 65536) {
    hipLaunchKernelGGL(permute_small_kernel<kSmallThreads>, dim3(1), dim3(kSmallThreads), wide_lds, s, p);
    return launched("permute_small_kernel");
  }
  if (slots <= kNarrowSmallSlots) {
    hipLaunchKernelGGL(permute_small_kernel<kPermuteThreads>, dim3(1), dim3(kPermuteThreads),
                       sizeof(int32_t) * ((kPermuteWaves + 1) * p.buckets + 1), s, p);
    return launched("permute_small_kernel");
  }
  hipLaunchKernelGGL(permute_count_kernel, dim3(p.blocks), dim3(kPermuteThreads), sizeof(int32_t) * p.buckets, s, p);
  if (int rc = launched("permute_count_kernel")) return rc;
  hipLaunchKernelGGL(permute_scan_kernel, dim3(1), dim3(kPermuteThreads), sizeof(int32_t) * (p.buckets + 1), s, p);
  if (int rc = launched("permute_scan_kernel")) return rc;
  hipLaunchKernelGGL(permute_scatter_kernel, dim3(p.blocks), dim3(kPermuteThreads),
                     sizeof(int32_t) * kPermuteWaves * p.buckets, s, p);
  return launched("permute_scatter_kernel");
}

static int permute_arguments(const char* who, const int32_t* indices, int32_t tokens, int32_t top_k, int32_t experts,
                             const int32_t* sizes, const int32_t* offsets, const int32_t* order, const int32_t* rows) {
  DEW_REQUIRE(tokens >= 0 && top_k >= 1, "%s: tokens %d top_k %d", who, tokens, top_k);
  DEW_REQUIRE(experts >= 1 && experts <= kMaxExperts, "%s: experts %d (at most %d)", who, experts, kMaxExperts);
  DEW_REQUIRE(static_cast<int64_t>(tokens) * top_k < (1ll << 30), "%s: %d x %d slots overflow int32", who, tokens, top_k);
  DEW_REQUIRE(sizes && offsets, "%s: sizes and offsets must not be null", who);
  DEW_REQUIRE(tokens * top_k == 0 || (indices && order && rows), "%s: indices, order and rows must not be null", who);
  return DEW_MOE_OK;
}

// The library's own scratch for dew_moe_permute_static: the per-block counts and bases of the three-launch sort.
// Every GPU the library runs on holds its own copy of the array until the process ends. The array's name is a
// host-side stand-in for it, not a device address: host code uses the address hipGetSymbolAddress returns for the
// current device, looked up once a device and kept.
constexpr size_t kStaticScratchBytes = DEW_MOE_PERMUTE_STATIC_BYTES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* scratch_of_device[kMaxDevices];  // null until the device's first call
static std::mutex scratch_lookup;

static int static_scratch(const char* who, void** out) {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
    return fail(DEW_MOE_EDEVICE, "%s: no HIP device below %d is current", who, kMaxDevices);
  std::lock_guard<std::mutex> hold(scratch_lookup);
  if (scratch_of_device[device] == nullptr) {
    void* address = nullptr;
    const hipError_t status = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (status != hipSuccess || address == nullptr)
      return fail(DEW_MOE_ELAUNCH, "%s: hipGetSymbolAddress of the scratch array on device %d: %s", who, device,
                  hipGetErrorString(status));
    scratch_of_device[device] = address;
  }
  *out = scratch_of_device[device];
  return DEW_MOE_OK;
}

}  // namespace dew

extern "C" int dew_moe_permute(const int32_t* indices, int32_t tokens, int32_t top_k, int32_t experts,
                               int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows,
                               void* workspace, size_t workspace_bytes, void* stream) {
  using namespace dew;
  if (int rc = permute_arguments("dew_moe_permute", indices, tokens, top_k, experts, sizes, offsets, order, rows)) return rc;
  const int slots = tokens * top_k;
  DEW_REQUIRE(workspace && workspace_bytes >= dew_moe_permute_workspace_bytes(slots, experts),
              "dew_moe_permute: workspace of %zu bytes, need %zu", workspace_bytes,
              dew_moe_permute_workspace_bytes(slots, experts));
  const uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + 255) & ~static_cast<uintptr_t>(255);
  return permute_launches(indices, tokens, top_k, experts, 0, sizes, offsets, order, rows, reinterpret_cast<int32_t*>(base),
                          static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_permute_shared(const int32_t* indices, int32_t tokens, int32_t top_k, int32_t experts, int32_t shared_rows,
                                      int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows, void* workspace,
                                      size_t workspace_bytes, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_permute_shared";
  if (int rc = permute_arguments(who, indices, tokens, top_k, experts, sizes, offsets, order, rows)) return rc;
  DEW_REQUIRE(shared_rows >= 0 && static_cast<int64_t>(tokens) * top_k + shared_rows < (1ll << 30) && experts < kMaxExperts,
              "%s: %d shared rows beside %d x %d slots, %d experts (a shared group needs one below %d)", who, shared_rows, tokens,
              top_k, experts, kMaxExperts);
  DEW_REQUIRE(shared_rows == 0 || (order && rows), "%s: order and rows must not be null", who);
  const int slots = tokens * top_k + shared_rows;
  const size_t need = dew_moe_permute_workspace_bytes(slots, experts + 1);
  DEW_REQUIRE(workspace && workspace_bytes >= need, "%s: workspace of %zu bytes, need %zu", who, workspace_bytes, need);
  const uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + 255) & ~static_cast<uintptr_t>(255);
  return permute_launches(indices, tokens, top_k, experts, shared_rows, sizes, offsets, order, rows, reinterpret_cast<int32_t*>(base),
                          static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_permute_static(const int32_t* indices, int32_t tokens, int32_t top_k, int32_t experts,
                                      int32_t* sizes, int32_t* offsets, int32_t* order, int32_t* rows, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_permute_static";
  if (int rc = permute_arguments(who, indices, tokens, top_k, experts, sizes, offsets, order, rows)) return rc;
  const size_t need = dew_moe_permute_workspace_bytes(tokens * top_k, experts);
  DEW_REQUIRE(need <= kStaticScratchBytes,
              "%s: %d slots over %d experts need %zu bytes of scratch, the library's own array holds %zu; use dew_moe_permute "
              "with a workspace", who, tokens * top_k, experts, need, kStaticScratchBytes);
  void* base = nullptr;
  if (int rc = static_scratch(who, &base)) return rc;
  // every int32 of the counts and bases a call reads is written earlier in the same call: nothing to clear
  return permute_launches(indices, tokens, top_k, experts, 0, sizes, offsets, order, rows, static_cast<int32_t*>(base),
                          static_cast<hipStream_t>(stream));
}

extern "C" int dew_moe_capacity_admit(const int32_t* indices, int32_t sequences, int32_t length, int32_t top_k, int32_t experts,
                                      int32_t capacity, int32_t* admitted, void* stream) {
  using namespace dew;
  const char* who = "dew_moe_capacity_admit";
  DEW_REQUIRE(sequences >= 0 && length >= 0 && top_k >= 1 && capacity >= 0, "%s: %d sequences of %d x %d slots, capacity %d", who,
              sequences, length, top_k, capacity);
  DEW_REQUIRE(experts >= 1 && experts <= kMaxExperts, "%s: experts %d (at most %d)", who, experts, kMaxExperts);
  DEW_REQUIRE(static_cast<int64_t>(sequences) * length * top_k < (1ll << 30), "%s: the slots overflow int32", who);
  if (sequences == 0 || length == 0) return DEW_MOE_OK;
  DEW_REQUIRE(indices && admitted, "%s: indices and admitted must not be null", who);
  hipLaunchKernelGGL(capacity_admit_kernel, dim3(sequences), dim3(kPermuteThreads), sizeof(int32_t) * kPermuteWaves * (experts + 1),
                     static_cast<hipStream_t>(stream), indices, admitted, length * top_k, experts, capacity);
  return launched("capacity_admit_kernel");
}
