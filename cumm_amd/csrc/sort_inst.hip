// Stable ascending sort of (mask & filter) with the permutation that does it: the step between
// the pair tables and the mask-based kernels (the reference's callers take it from spconv's
// sort_1d_by_key[_split], cumm/conv/main_real_spconv.py:118-145).
//
// Least-significant-digit radix sort, 9 bits per pass (three passes for the 27 offsets of a
// 3 x 3 x 3 kernel), one kernel per pass plus one kernel in front:
//   * sort_setup_kernel reads the keys once and makes the histograms of ALL passes (the digits of
//     a key do not depend on the order the keys are in), clears the look-back state and the block
//     tickets;
//   * a pass whose digit is the same in every key (the histogram shows it: the bits of a 32-bit
//     filter above the kernel volume, any pass of an input with one mask value) moves nothing: its
//     workgroups leave at once, and the passes that do move keys work out among themselves which
//     of the two buffers each reads and writes so that the last of them writes the caller's;
//   * a pass kernel is a single sweep: a workgroup takes the next chunk of 4096 keys (by ticket,
//     so that a chunk's predecessors have always started), ranks its keys per digit - per wave
//     by ballot matching, in position order, which is what makes the pass stable -, publishes its
//     per-digit counts, finds the counts of all chunks before it by looking back over what they
//     have published (a chunk publishes its own counts at once and the running total when it
//     knows it; a look-back stops at the first running total), and scatters.
//   * sort_finish_kernel, behind the last pass, counts the light prefix of the sorted array into
//     the hint slot that a later convolution launch on this array looks up (launch.h).
// Every spin on another workgroup's state is bounded: a wave that gives up counts itself and goes
// on, so the grid always drains.  The finish kernel then replaces the result by the identity
// order (argsort = 0 .. n-1, the masks as they came): any permutation with its masks is a valid
// input of the convolution kernels - the order only decides how light the tiles are - so what
// follows on the stream computes the right thing, slowly, and the host reports the give-up at
// its next synchronisation.
// Integer work, bound by launch latency at 10^5 keys and by HBM / L2 traffic at 10^6 and more.
#include "launch.h"
#include "lds_dma.h"

namespace cummhip {

namespace {

constexpr int kRadixBits = 9;
constexpr int kBins = 1 << kRadixBits;            // 512
constexpr int kSortThreads = 512;                 // one bin per thread
constexpr int kSortWaves = kSortThreads / 64;     // 8
constexpr int kItems = 8;                         // keys per lane: 4096 keys per workgroup of a pass ...
// ... and half of that for inputs of up to kSmallInput keys, where the chunks are few and a pass is
// as long as one chunk's chain of round trips (120 k keys: 62.7 us with 59 chunks of 2048 against
// 70.8 us with 30 of 4096; at 1 M keys the larger chunks win, 131 against 152 us)
constexpr int kSmallItems = 4;
constexpr int kSmallInput = 1 << 18;
inline int pass_items(int n) { return n <= kSmallInput ? kSmallItems : kItems; }
constexpr uint32_t kFlagAggregate = 1u << 30, kFlagInclusive = 2u << 30, kValueMask = (1u << 30) - 1u;
constexpr int kLookbackSpins = 1 << 20;   // (about a second)

struct SortParams {
  const uint32_t *mask;      // [n] the caller's masks
  uint32_t filter;
  int32_t n, chunks, passes;
  uint32_t *hist;            // [passes][kBins] keys per digit value
  uint32_t *state;           // [passes][chunks][kBins] look-back words
  uint32_t *tickets;         // [passes] next chunk to hand out
  int32_t *give_ups;         // counts the look-backs that ran into their bound (the host reports them)
  int32_t pass;
  uint32_t *out_keys, *tmp_keys;   // the caller's arrays and the workspace's: the passes alternate between them
  int32_t *out_vals, *tmp_vals;
  int32_t *hint_slot;        // light-prefix hint of the sorted array (launch.h), or NULL
  // 0: ascending mask value (spconv's sort_1d_by_key).  1: ascending number of kernel offsets, then
  // ascending value (the filter has at most kCountShift significant bits): positions of few
  // offsets first, the few of many offsets last - tiles of the heavy end then OR together masks
  // of similar weight, and the many-offset tiles of a launch form a short run at its end.
  int32_t count_major;
};

constexpr int kCountShift = 27;
// sort key of a mask word
__device__ __forceinline__ uint32_t sort_key(const SortParams &p, uint32_t mask_word) {
  const uint32_t m = mask_word & p.filter;
  return p.count_major ? ((uint32_t)__builtin_popcount(m) << kCountShift) | m : m;
}
// ... and the mask word back out of it
__device__ __forceinline__ uint32_t key_mask(const SortParams &p, uint32_t key) {
  return p.count_major ? key & ((1u << kCountShift) - 1u) : key;
}

__global__ __launch_bounds__(kSortThreads) void sort_setup_kernel(const SortParams p) {
  __shared__ uint32_t lds_hist[4][kBins];
  const int t = threadIdx.x;
  for (int q = 0; q < p.passes; ++q) lds_hist[q][t] = 0u;
  // look-back state and tickets start at zero (the workspace holds whatever was there)
  const size_t words = (size_t)p.passes * p.chunks * kBins;
  for (size_t i = (size_t)blockIdx.x * kSortThreads + t; i < words; i += (size_t)gridDim.x * kSortThreads) p.state[i] = 0u;
  if (blockIdx.x == 0 && t < p.passes) p.tickets[t] = 0u;
  if (blockIdx.x == 0 && t < 8 && p.hint_slot != nullptr)   // names no array yet; the two counts start at "everything" / "nothing"
    p.hint_slot[t] = t == 4 ? (p.n / 128) * 128 : (t == 5 ? ((p.n + 63) / 64) * 64 : 0);
  __syncthreads();
  // lanes of a wave with the same digit add once (most masks of a sparse cloud are the same word:
  // one add per lane would queue 64 deep on one LDS address)
  const int lane = t & 63;
  const int64_t span = (int64_t)gridDim.x * kSortThreads;
  const int64_t rounds = (p.n + span - 1) / span;
  for (int64_t r0 = 0; r0 < rounds; r0 += kItems) {
    // kItems keys per lane are requested together (one memory round trip, not one per key)
    uint32_t keys[kItems];
    bool valids[kItems];
#pragma unroll
    for (int u = 0; u < kItems; ++u) {
      const int64_t i = (r0 + u) * span + (int64_t)blockIdx.x * kSortThreads + t;
      valids[u] = r0 + u < rounds && i < p.n;
      keys[u] = valids[u] ? sort_key(p, p.mask[i]) : 0u;
    }
#pragma unroll
    for (int u = 0; u < kItems; ++u) {
      // a wave whose 64 keys are one word (the centre-only masks of a sparse cloud: most waves) adds
      // once per digit without looking for its peers
      const unsigned long long live = __ballot(valids[u]);
      if (live == 0ull) continue;
      const uint32_t first_key = (uint32_t)__builtin_amdgcn_readlane((int)keys[u], __builtin_ctzll(live));
      if (__ballot(valids[u] && keys[u] == first_key) == live) {
        if (lane < p.passes)
          atomicAdd(&lds_hist[lane][(first_key >> (lane * kRadixBits)) & (kBins - 1)], (uint32_t)__popcll(live));
        continue;
      }
      for (int q = 0; q < p.passes; ++q) {
        const uint32_t d = (keys[u] >> (q * kRadixBits)) & (kBins - 1);
        unsigned long long peers = __ballot(valids[u]);
#pragma unroll
        for (int b = 0; b < kRadixBits; ++b) {
          const unsigned long long has = __ballot((d >> b) & 1u);
          peers &= ((d >> b) & 1u) ? has : ~has;
        }
        if (valids[u] && (peers & ((1ull << lane) - 1ull)) == 0ull) atomicAdd(&lds_hist[q][d], (uint32_t)__popcll(peers));
      }
    }
  }
  __syncthreads();
  for (int q = 0; q < p.passes; ++q) {
    const uint32_t c = lds_hist[q][t];
    if (c) atomicAdd(&p.hist[q * kBins + t], c);
  }
}

// (the histograms are accumulated with atomics: they start from zero in a kernel of their own
// stream order before the setup kernel - see launch_sort_by_mask)
__global__ __launch_bounds__(256) void sort_clear_hist_kernel(uint32_t *hist, int words) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < words) hist[i] = 0u;
}

template <int ITEMS>
__global__ __launch_bounds__(kSortThreads) void sort_pass_kernel(const SortParams p) {
  constexpr int kChunk = kSortThreads * ITEMS;
  __shared__ uint32_t wave_hist[kSortWaves][kBins];   // per wave: keys per digit, then the prefix over waves
  __shared__ uint32_t bin_base[kBins];                // where this chunk's keys of a digit go
  __shared__ uint32_t scan_tmp[kBins];
  __shared__ int chunk_of_block;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int shift = p.pass * kRadixBits;

  // which passes move keys at all (thread = bin: a bin that holds every key makes its pass idle)
  uint32_t tot[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) tot[q] = q < p.passes ? p.hist[q * kBins + t] : (t == 0 ? (uint32_t)p.n : 0u);
  int movers = 0, movers_before = 0;
  bool mine_moves = false;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const bool idle = __syncthreads_or(tot[q] == (uint32_t)p.n) != 0;
    if (!idle) {
      ++movers;
      if (q < p.pass) ++movers_before;
      if (q == p.pass) mine_moves = true;
    }
  }
  // nothing moves at all (one mask value): the first pass copies the input through
  const bool copy_through = movers == 0 && p.pass == 0;
  if (!mine_moves && !copy_through) return;
  // the last mover writes the caller's arrays, the ones before it alternate; the first one
  // reads the caller's masks (and the identity order)
  const bool first = movers_before == 0;
  const bool last = movers - 1 - movers_before == 0;
  const bool to_out = copy_through || ((movers - 1 - movers_before) & 1) == 0;
  uint32_t *const dst_keys = to_out ? p.out_keys : p.tmp_keys;
  int32_t *const dst_vals = to_out ? p.out_vals : p.tmp_vals;
  const uint32_t *const src_keys = to_out ? p.tmp_keys : p.out_keys;
  const int32_t *const src_vals = to_out ? p.tmp_vals : p.out_vals;
  // chunks are handed out by ticket: a chunk's predecessors have then always started, whatever
  // order the workgroups are dispatched in and however many of them are resident
  if (t == 0) chunk_of_block = (int)atomicAdd(&p.tickets[p.pass], 1u);
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) wave_hist[w][t] = 0u;
  // exclusive prefix over the digit values of the whole input: thread = bin; a scan inside each
  // wave by lane shuffles, then the totals of the waves before
  const uint32_t total_of_bin = p.pass == 0 ? tot[0] : (p.pass == 1 ? tot[1] : (p.pass == 2 ? tot[2] : tot[3]));
  uint32_t incl = total_of_bin;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
    if (lane >= off) incl += up;
  }
  if (lane == 63) scan_tmp[wave] = incl;
  __syncthreads();
  uint32_t waves_before = 0;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) waves_before += w < wave ? scan_tmp[w] : 0u;
  const uint32_t global_excl = waves_before + incl - total_of_bin;
  const int chunk = chunk_of_block;
  if (chunk >= p.chunks) return;   // (never: the grid has one workgroup per chunk)

  if (copy_through) {
#pragma unroll
    for (int u = 0; u < ITEMS; ++u) {
      const int64_t pos = (int64_t)chunk * kChunk + u * kSortThreads + t;
      if (pos < p.n) {
        dst_keys[pos] = p.mask[pos] & p.filter;      // (nothing moves: the masks themselves)
        dst_vals[pos] = (int32_t)pos;
      }
    }
    return;
  }

  // ---- keys of this chunk, wave-striped: wave w owns positions [base_w, base_w + 64 * ITEMS),
  // item u of lane l is position base_w + u * 64 + l, i.e. position order = (u, l)
  const int64_t base_w = (int64_t)chunk * kChunk + (int64_t)wave * (64 * ITEMS);
  uint32_t key[ITEMS];
  int32_t val[ITEMS];
  uint32_t rank[ITEMS];   // offset among this wave's keys of the same digit
#pragma unroll
  for (int u = 0; u < ITEMS; ++u) {
    const int64_t pos = base_w + u * 64 + lane;
    const bool valid = pos < p.n;
    if (first) {
      key[u] = valid ? sort_key(p, p.mask[pos]) : 0u;
      val[u] = (int32_t)pos;
    } else {
      key[u] = valid ? src_keys[pos] : 0u;
      val[u] = valid ? src_vals[pos] : 0;
    }
  }
#pragma unroll
  for (int u = 0; u < ITEMS; ++u) {
    const int64_t pos = base_w + u * 64 + lane;
    const bool valid = pos < p.n;
    const uint32_t d = (key[u] >> shift) & (kBins - 1);
    // lanes with the same digit (positions past the end match nobody)
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int b = 0; b < kRadixBits; ++b) {
      const unsigned long long has = __ballot((d >> b) & 1u);
      peers &= ((d >> b) & 1u) ? has : ~has;
    }
    const uint32_t before = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
    uint32_t prev = 0;
    if (valid) prev = wave_hist[wave][d];
    __builtin_amdgcn_wave_barrier();
    if (valid && before == 0) wave_hist[wave][d] = prev + (uint32_t)__popcll(peers);
    __builtin_amdgcn_wave_barrier();
    rank[u] = prev + before;
  }
  __syncthreads();

  // ---- thread = bin: prefix over the waves, this chunk's count, look-back over the chunks before
  uint32_t count = 0;
#pragma unroll
  for (int w = 0; w < kSortWaves; ++w) {
    const uint32_t c = wave_hist[w][t];
    wave_hist[w][t] = count;
    count += c;
  }
  uint32_t *my_state = p.state + ((size_t)p.pass * p.chunks + chunk) * kBins;
  // (relaxed device-scope stores: the word itself carries flag and value, nothing else is published
  // through it; a release here writes back the whole L2 of the XCD, once per wave)
  __hip_atomic_store(&my_state[t], (chunk == 0 ? kFlagInclusive : kFlagAggregate) | count, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
  uint32_t before_chunks = 0;
  if (chunk > 0) {
    // Look back over the chunks before this one, kLook of them per round trip: the words of a
    // batch are requested together (the word carries flag and value, so relaxed loads do), then
    // taken in order until a running total ends the walk; a word that is not there yet is asked
    // for again, from there.  One thread walking one predecessor per round trip made a pass of
    // 30 chunks take 45 us.
    constexpr int kLook = 16;
    bool gave_up = false, done = false;
    int j = chunk - 1, spins = 0;
    while (!done && !gave_up) {
      uint32_t sw[kLook];
#pragma unroll
      for (int i = 0; i < kLook; ++i) {
        const int c = j - i;
        sw[i] = c >= 0 ? __hip_atomic_load(p.state + ((size_t)p.pass * p.chunks + c) * kBins + t, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT)
                       : kFlagInclusive;
      }
      int taken = 0;
#pragma unroll
      for (int i = 0; i < kLook; ++i) {
        if (!done && taken == i) {
          const uint32_t flag = sw[i] >> 30;
          if (flag != 0u) {
            before_chunks += sw[i] & kValueMask;
            ++taken;
            if (flag == 2u) done = true;
          }
        }
      }
      j -= taken;
      if (!done && taken == 0) {
        if (++spins > kLookbackSpins) gave_up = true;
        __builtin_amdgcn_s_sleep(2);
      }
    }
    if (gave_up && p.give_ups != nullptr) atomicAdd(p.give_ups, 1);
    __hip_atomic_store(&my_state[t], kFlagInclusive | (before_chunks + count), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  bin_base[t] = global_excl + before_chunks;
  __syncthreads();

  // ---- scatter
#pragma unroll
  for (int u = 0; u < ITEMS; ++u) {
    const int64_t pos = base_w + u * 64 + lane;
    if (pos < p.n) {
      const uint32_t d = (key[u] >> shift) & (kBins - 1);
      const uint32_t dst = bin_base[d] + wave_hist[wave][d] + rank[u];
      dst_keys[dst] = last ? key_mask(p, key[u]) : key[u];     // the caller gets masks, not keys
      dst_vals[dst] = val[u];
    }
  }
}

// What a later launch can use about a sorted mask array, counted here into its hint slot:
//   * the light prefix (slot word 4): the number of leading runs of 128 positions whose two halves
//     of 64 each have at most `light` kernel offsets in the OR of their masks, as a number of
//     positions - those go to 128-row tiles.  `light` is 2 for the order by value; in the order by
//     offset count the runs of equal two-offset masks follow one another, and the tile at each
//     seam has three: 3 there.
//   * where the heavy end begins (slot word 5): the first tile of 64 positions with kHeavyOffsets or
//     more kernel offsets, as a position - a launch may take the tiles from there on in halves of
//     32 rows when they are few (in the order by offset count they are the last few tiles).
// One wave per run of 128; a run that fails lowers a count that starts at "all" / "none".
constexpr int kLightOffsets = 2, kLightOffsetsByCount = 3, kHeavyOffsets = 10;

__global__ __launch_bounds__(64) void light_prefix_init_kernel(int32_t *result, int32_t *hint_slot, int n) {
  if (threadIdx.x == 0 && result != nullptr) *result = (n / 128) * 128;
  if (threadIdx.x < 8 && hint_slot != nullptr)
    hint_slot[threadIdx.x] = threadIdx.x == 4 ? (n / 128) * 128 : (threadIdx.x == 5 ? ((n + 63) / 64) * 64 : 0);
}

// Names the array a hint slot describes (the counts have been lowered by then or are being lowered
// by the same kernel: a launch that reads the slot comes later on the stream).
__device__ __forceinline__ void name_hint_slot(int32_t *slot, const uint32_t *sorted, int n, uint32_t filter) {
  const uint64_t a = (uint64_t)sorted;
  slot[0] = (int32_t)(uint32_t)a;
  slot[1] = (int32_t)(uint32_t)(a >> 32);
  slot[2] = n;
  slot[3] = (int32_t)filter;
}

// one wave, one run of 128 positions (the last run may be short: it only counts for the heavy end)
__device__ __forceinline__ void count_run(const uint32_t *sorted, int n, uint32_t filter, int run, int lane, int light,
                                          int32_t *result, int32_t *hint_slot) {
  const int64_t p0 = (int64_t)run * 128 + lane, p1 = p0 + 64;
  const uint32_t lo = wave_or_dpp(p0 < n ? sorted[p0] & filter : 0u);
  const uint32_t hi = wave_or_dpp(p1 < n ? sorted[p1] & filter : 0u);
  if (lane != 0) return;
  const int c0 = __builtin_popcount(lo), c1 = __builtin_popcount(hi);
  if (run < n / 128 && (c0 > light || c1 > light)) {
    if (result != nullptr) atomicMin(result, run * 128);
    if (hint_slot != nullptr) atomicMin(&hint_slot[4], run * 128);
  }
  if (hint_slot != nullptr && (c0 >= kHeavyOffsets || c1 >= kHeavyOffsets))
    atomicMin(&hint_slot[5], run * 128 + (c0 >= kHeavyOffsets ? 0 : 64));
}

__global__ __launch_bounds__(256) void light_prefix_kernel(const uint32_t *sorted, int n, uint32_t filter,
                                                           int32_t *result, int32_t *hint_slot) {
  const int lane = threadIdx.x & 63;
  const int run = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (blockIdx.x == 0 && threadIdx.x == 0 && hint_slot != nullptr) name_hint_slot(hint_slot, sorted, n, filter);
  if ((int64_t)run * 128 >= n) return;
  count_run(sorted, n, filter, run, lane, kLightOffsets, result, hint_slot);
}

// Behind the last pass of the sort: the counts of the result into the hint slot - or, when a
// look-back of this device has given up since the host last looked, the identity order in place
// of a result that cannot be trusted.  One wave per 128 positions, the last run may be short.
__global__ __launch_bounds__(256) void sort_finish_kernel(const SortParams p) {
  const int lane = threadIdx.x & 63;
  const int run = blockIdx.x * 4 + (threadIdx.x >> 6);
  const bool broken = p.give_ups != nullptr && __hip_atomic_load(p.give_ups, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
  if (broken) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int64_t pos = (int64_t)run * 128 + h * 64 + lane;
      if (pos < p.n) {
        p.out_keys[pos] = p.mask[pos] & p.filter;
        p.out_vals[pos] = (int32_t)pos;
      }
    }
    if (p.hint_slot != nullptr && blockIdx.x == 0 && threadIdx.x < 8) p.hint_slot[threadIdx.x] = 0;
    return;
  }
  if (p.hint_slot == nullptr) return;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    name_hint_slot(p.hint_slot, p.out_keys, p.n, p.filter);
    p.hint_slot[6] = p.count_major;
  }
  if ((int64_t)run * 128 >= p.n) return;
  count_run(p.out_keys, p.n, 0xFFFFFFFFu, run, lane, p.count_major ? kLightOffsetsByCount : kLightOffsets, nullptr, p.hint_slot);
}

size_t align256s(size_t x) { return (x + 255) & ~(size_t)255; }

int sort_passes(uint32_t filter) {
  int end_bit = 32;
  while (end_bit > 1 && !((filter >> (end_bit - 1)) & 1u)) --end_bit;
  return (end_bit + kRadixBits - 1) / kRadixBits;   // 1 .. 4
}

}  // namespace

// keys + values of the intermediate order, histograms, tickets, look-back state
size_t sort_by_mask_workspace_bytes(int n) {
  const size_t nn = (size_t)(n > 0 ? n : 1);
  const size_t chunk = (size_t)kSortThreads * pass_items((int)nn);
  size_t chunks = (nn + chunk - 1) / chunk;
  // (never less than a smaller input asks for: a workspace sized for a larger one must do)
  const size_t small_most = ((size_t)kSmallInput + kSortThreads * kSmallItems - 1) / (kSortThreads * kSmallItems);
  if (nn > (size_t)kSmallInput && chunks < small_most) chunks = small_most;
  return 2 * align256s(4 * nn) + align256s(4 * 4 * kBins) + 256 + align256s(4 * 4 * chunks * kBins);
}

hipError_t launch_sort_by_mask(const uint32_t *mask, int n, uint32_t filter, uint32_t *sorted, int32_t *argsort,
                               void *workspace, int32_t *give_ups, int32_t *hint_slot, int order, hipStream_t s) {
  if (n <= 0) return hipSuccess;
  if (order != 0 && (filter >> kCountShift) != 0u) return hipErrorInvalidValue;   // no room for the count above the mask
  char *base = reinterpret_cast<char *>(workspace);
  const size_t words = align256s(4 * (size_t)n);
  SortParams p;
  p.mask = mask; p.filter = filter; p.n = n;
  const int items = pass_items(n), chunk = kSortThreads * items;
  p.chunks = (n + chunk - 1) / chunk;
  p.count_major = order != 0;
  p.passes = p.count_major ? 4 : sort_passes(filter);
  p.out_keys = sorted; p.out_vals = argsort;
  p.tmp_keys = reinterpret_cast<uint32_t *>(base);
  p.tmp_vals = reinterpret_cast<int32_t *>(base + words);
  p.hist = reinterpret_cast<uint32_t *>(base + 2 * words);
  p.tickets = reinterpret_cast<uint32_t *>(base + 2 * words + align256s(4 * 4 * kBins));
  p.state = reinterpret_cast<uint32_t *>(base + 2 * words + align256s(4 * 4 * kBins) + 256);
  p.give_ups = give_ups;
  p.hint_slot = hint_slot;
  p.pass = 0;
  hipLaunchKernelGGL(sort_clear_hist_kernel, dim3((4 * kBins + 255) / 256), dim3(256), 0, s, p.hist, 4 * kBins);
  // (two keys per lane where that still leaves fewer workgroups than the device holds: with one
  // workgroup per chunk the 120 k keys of a small input sat on 30 or 59 of the 256 CUs)
  int setup_blocks = (n + 2 * kSortThreads - 1) / (2 * kSortThreads);
  if (setup_blocks > 512) setup_blocks = 512;
  hipLaunchKernelGGL(sort_setup_kernel, dim3(setup_blocks), dim3(kSortThreads), 0, s, p);
  for (int q = 0; q < p.passes; ++q) {
    SortParams r = p;
    r.pass = q;
    if (items == kSmallItems) hipLaunchKernelGGL(sort_pass_kernel<kSmallItems>, dim3(p.chunks), dim3(kSortThreads), 0, s, r);
    else hipLaunchKernelGGL(sort_pass_kernel<kItems>, dim3(p.chunks), dim3(kSortThreads), 0, s, r);
  }
  hipLaunchKernelGGL(sort_finish_kernel, dim3((n + 511) / 512), dim3(256), 0, s, p);
  return hipGetLastError();
}

hipError_t launch_light_prefix(const uint32_t *sorted, int n, uint32_t filter, int32_t *result, int32_t *hint_slot,
                               hipStream_t s) {
  const int runs = (n + 127) / 128;
  hipLaunchKernelGGL(light_prefix_init_kernel, dim3(1), dim3(64), 0, s, result, hint_slot, n);
  hipLaunchKernelGGL(light_prefix_kernel, dim3(runs > 0 ? (runs + 3) / 4 : 1), dim3(256), 0, s, sorted, n, filter, result,
                     hint_slot);
  return hipGetLastError();
}

}  // namespace cummhip
