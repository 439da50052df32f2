// Pair tables of a submanifold convolution, on the GPU: the step right before
// the mask-based kernels (the reference's callers get it from spconv's generate_subm_conv_inds and
// sort_1d_by_key, cumm/conv/main_real_spconv.py:91-145; the reference's own building block is the
// linear-probing LinearHashTable of include/tensorview/hash/linear.cu.h:111-840).
//
//   indices_fwd[k][o] = row of the voxel at coord[o] + (k_zyx - center) * dilation, or -1
//   mask_fwd[o]       = OR of (1 << k) over the offsets with a pair
//   indices_bwd[k]    = indices_fwd[kv-1-k],  mask_bwd = mask_fwd with its kv bits reversed
//
// The table depends on the geometry only, never on the hash, so it is bit-exact against the host
// builder whatever the hash.  Integer work, bound by HBM / L2 traffic:
//   * open addressing with linear probing over 16-byte slots {64-bit key, row}: one load returns
//     both, the table of 2N..4N slots (2-4 MB at 120 k voxels) stays in L2;
//   * in front of the table sits a hashed presence bitmap, one 32-bit word per run of 32 sites
//     along x (1 MB at 120 k voxels, L2-resident): most look-ups of a sparse cloud are misses,
//     and the word turns them away - all x-neighbours of a row with one load - before they cost
//     table sectors;
//   * the lookup kernel is one lane per (voxel, (kz, ky)): for a fixed offset consecutive lanes
//     write consecutive table entries (coalesced).  Measured at 120 k voxels: one lane per voxel
//     walking its 27 offsets 127 us, one lane per (voxel, offset) without the bitmap 66 us;
#include <hip/hip_runtime.h>

#include <cstring>


#include "launch.h"

namespace cummhip {

namespace {

struct __attribute__((aligned(16))) Slot {
  unsigned long long key;
  int32_t row;
  int32_t pad;
};
constexpr unsigned long long kEmptyKey = ~0ull;

__device__ __forceinline__ unsigned long long mix64(unsigned long long k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdull;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ull;
  k ^= k >> 33;
  return k;
}

// one launch empties the table, the presence words and the masks
__global__ __launch_bounds__(256) void pairs_clear_kernel(const SubmPairsParams p) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i <= p.slot_mask) reinterpret_cast<Slot *>(p.table)[i] = Slot{kEmptyKey, -1, 0};
  if (i <= p.filter_mask) p.filter[i] = 0u;
  if (i < (uint32_t)p.n) {
    // every voxel pairs with itself through the centre offset: that bit is set here, and the
    // look-up kernel neither probes the table nor touches the masks for it
    if (p.mask_f) p.mask_f[i] = p.center_k >= 0 ? 1u << p.center_k : 0u;
    if (p.mask_b) p.mask_b[i] = p.center_k >= 0 ? 1u << (p.kv - 1 - p.center_k) : 0u;
  }
}

__device__ __forceinline__ unsigned long long coord_key(int b, int z, int y, int x, const SubmPairsParams &p) {
  return (((unsigned long long)b * p.shape[0] + z) * p.shape[1] + y) * p.shape[2] + x;
}
// presence word of the 32 sites (b, z, y, 32*(x/32) ..): hashed, without a key, so a set bit
// means "maybe" (two runs may share a word) and a clear bit means "certainly absent"
__device__ __forceinline__ uint32_t presence_index(int b, int z, int y, int x, const SubmPairsParams &p) {
  const unsigned long long run = (((unsigned long long)b * p.shape[0] + z) * p.shape[1] + y) * ((p.shape[2] + 31) >> 5) + (x >> 5);
  return (uint32_t)mix64(run ^ 0x9e3779b97f4a7c15ull) & p.filter_mask;
}

__global__ __launch_bounds__(256) void pairs_insert_kernel(const SubmPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= p.n) return;
  const int4 c = reinterpret_cast<const int4 *>(p.coords)[i];
  const unsigned long long key = coord_key(c.x, c.y, c.z, c.w, p);
  Slot *table = reinterpret_cast<Slot *>(p.table);
  atomicOr(&p.filter[presence_index(c.x, c.y, c.z, c.w, p)], 1u << (c.w & 31));
  uint32_t h = (uint32_t)mix64(key) & p.slot_mask;
  // at most `slots` probes: the table has at least twice as many slots as voxels
  for (uint32_t probe = 0; probe <= p.slot_mask; ++probe) {
    const unsigned long long prev = atomicCAS(&table[h].key, kEmptyKey, key);
    if (prev == kEmptyKey || prev == key) {
      table[h].row = i;   // (coordinates are unique: the caller's contract, as in spconv)
      break;
    }
    h = (h + 1) & p.slot_mask;
  }
}

// One lane per (voxel, (kz, ky)): it walks the KX offsets along x.  19 of 20 look-ups of a sparse
// cloud are misses, and a miss in the table costs two or more 64-byte sectors; the presence word
// of the neighbour's run of 32 sites answers all of a row's x-neighbours with one 4-byte load from
// a table that stays in L2, and only "maybe" goes on to the hash table.  grid.y = KZ*KY,
// consecutive lanes = consecutive voxels: every table row is written coalesced.  The masks are
// OR-ed with atomics, one per PAIR, into words that the clear kernel zeroed.
__global__ __launch_bounds__(256) void pairs_lookup_kernel(const SubmPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int zy = blockIdx.y;
  if (i >= p.n) return;
  const int4 c = reinterpret_cast<const int4 *>(p.coords)[i];
  const Slot *table = reinterpret_cast<const Slot *>(p.table);
  uint32_t have_index = ~0u, word = 0;
  for (int kx = 0; kx < p.kx; ++kx) {
    const int k = zy * p.kx + kx;
    if (k == p.center_k) {
      p.ind_f[(int64_t)k * p.n + i] = i;
      if (p.ind_b) p.ind_b[(int64_t)(p.kv - 1 - k) * p.n + i] = i;
      continue;
    }
    const int z = c.y + p.off[k][0], y = c.z + p.off[k][1], x = c.w + p.off[k][2];
    int row = -1;
    if (z >= 0 && z < p.shape[0] && y >= 0 && y < p.shape[1] && x >= 0 && x < p.shape[2]) {
      const uint32_t index = presence_index(c.x, z, y, x, p);
      if (index != have_index) {
        word = p.filter[index];
        have_index = index;
      }
      if ((word >> (x & 31)) & 1u) {
        const unsigned long long key = coord_key(c.x, z, y, x, p);
        uint32_t h = (uint32_t)mix64(key) & p.slot_mask;
        Slot s = table[h];
        // a collision walks on until the key or an empty slot turns up (the table is never full)
        for (uint32_t probe = 0; s.key != key && s.key != kEmptyKey && probe <= p.slot_mask; ++probe) {
          h = (h + 1) & p.slot_mask;
          s = table[h];
        }
        if (s.key == key) row = s.row;
      }
    }
    p.ind_f[(int64_t)k * p.n + i] = row;
    if (p.ind_b) p.ind_b[(int64_t)(p.kv - 1 - k) * p.n + i] = row;
    if (row >= 0) {
      if (p.mask_f) atomicOr(&p.mask_f[i], 1u << k);
      if (p.mask_b) atomicOr(&p.mask_b[i], 1u << (p.kv - 1 - k));
    }
  }
}

// ---- regular (strided) sparse convolution: an output site is active iff an input falls into
// its receptive field; output rows are the active sites in ascending (batch, z, y, x) order.
// (What spconv's generate_conv_inds_mask_stage1 / unique / stage2 give the reference's callers.)
//   1. every (input, offset) computes its output site; the sites go into a hash set, whose keys
//      are then gathered into a list (one counter update per 8192 slots);
//   2. the list is sorted (radix sort over the bits of the largest key): position = output row;
//   3. the rows are written back into the set, and every (input, offset) looks its site up again:
//      indices_fwd[k][row] = input, indices_bwd[k][input] = row, the masks by atomic OR.
// The tables depend on the geometry only: bit-exact against the host builder.

// output site of input c through offset k: (c + pad - k*dilation) / stride where that is exact
__device__ __forceinline__ bool conv_out_site(const ConvPairsParams &p, const int4 c, int k, unsigned long long *key) {
  const int in[3] = {c.y, c.z, c.w};
  if (c.x < 0 || c.x >= p.batch) return false;
  unsigned long long acc = (unsigned long long)c.x;
#pragma unroll
  for (int d = 0; d < 3; ++d) {
    const int num = in[d] + p.pad[d] - p.koff[k][d];
    const int q = num / p.stride[d];
    if (num < 0 || q * p.stride[d] != num || q >= p.out_shape[d]) return false;
    acc = acc * (unsigned long long)p.out_shape[d] + (unsigned long long)q;
  }
  *key = acc;
  return true;
}

__global__ __launch_bounds__(256) void conv_pairs_clear_kernel(const ConvPairsParams p) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i <= p.slot_mask) reinterpret_cast<Slot *>(p.table)[i] = Slot{kEmptyKey, -1, 0};
  if (i < 2) p.counters[i] = 0ull;
}

__global__ __launch_bounds__(256) void conv_pairs_sites_kernel(const ConvPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (i >= p.n_in) return;
  Slot *table = reinterpret_cast<Slot *>(p.table);
  unsigned long long key = 0;
  if (!conv_out_site(p, reinterpret_cast<const int4 *>(p.coords)[i], k, &key)) return;
  uint32_t h = (uint32_t)mix64(key) & p.slot_mask;
  // most candidates repeat a site that is already there: look before the compare-and-swap (a
  // key never changes once set, so a stale look only costs the swap)
  for (uint32_t probe = 0; probe <= p.slot_mask; ++probe) {
    unsigned long long cur = __atomic_load_n(&table[h].key, __ATOMIC_RELAXED);
    if (cur == kEmptyKey) cur = atomicCAS(&table[h].key, kEmptyKey, key);
    if (cur == kEmptyKey || cur == key) break;
    h = (h + 1) & p.slot_mask;
  }
}

// The set's keys, gathered into a list in any order (it is sorted next).  A workgroup takes 8192
// slots and updates the shared counter and the shared maximum once each: updates of one address
// from all over the chip complete one at a time, about 6 ns each (one per wave of candidates, 250 k
// of them, took 1.5 ms; one per 2048 slots plus a maximum per wave 96 us).
constexpr int kCompactPerThread = 32;
__global__ __launch_bounds__(256) void conv_pairs_compact_kernel(const ConvPairsParams p) {
  __shared__ uint32_t wave_cnt[4];
  __shared__ unsigned long long wave_top[4];
  __shared__ unsigned long long wg_base;
  const Slot *table = reinterpret_cast<const Slot *>(p.table);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t first = blockIdx.x * (256u * kCompactPerThread);
  unsigned long long keys[kCompactPerThread];
  uint32_t mine = 0;
  unsigned long long top = 0;
#pragma unroll
  for (int u = 0; u < kCompactPerThread; ++u) {
    const uint32_t slot = first + (uint32_t)u * 256u + (uint32_t)tid;
    keys[u] = slot <= p.slot_mask ? table[slot].key : kEmptyKey;
  }
#pragma unroll
  for (int u = 0; u < kCompactPerThread; ++u) {
    const bool have = keys[u] != kEmptyKey;
    mine += (uint32_t)__popcll(__ballot(have));
    if (have && keys[u] > top) top = keys[u];
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    const unsigned long long other = __shfl_xor(top, off);
    top = other > top ? other : top;
  }
  if (lane == 0) {
    wave_cnt[wave] = mine;
    wave_top[wave] = top;
  }
  __syncthreads();
  if (tid == 0) {
    const uint32_t total = wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
    unsigned long long t = wave_top[0];
    for (int w = 1; w < 4; ++w) t = wave_top[w] > t ? wave_top[w] : t;
    wg_base = total ? atomicAdd(&p.counters[0], (unsigned long long)total) : 0ull;
    if (total) atomicMax(&p.counters[1], t);   // largest key: it bounds the sort's passes
  }
  __syncthreads();
  unsigned long long at = wg_base;
  for (int w = 0; w < wave; ++w) at += wave_cnt[w];
#pragma unroll
  for (int u = 0; u < kCompactPerThread; ++u) {
    const bool have = keys[u] != kEmptyKey;
    const unsigned long long found = __ballot(have);
    if (have) p.uniq[at + __popcll(found & ((1ull << lane) - 1ull))] = keys[u];
    at += __popcll(found);
  }
}

// every (row, offset) starts at -1; the sites get their rows, the coordinates are decoded and the
// masks zeroed
__global__ __launch_bounds__(256) void conv_pairs_rows_kernel(const ConvPairsParams p) {
  const int j = blockIdx.x * 256 + threadIdx.x;
  {
    // the whole forward table starts at -1: 16-byte stores over the flat array, the last thread
    // writes the odd words at the end
    const int64_t words = (int64_t)p.kv * p.n_out, quads = words >> 2;
    const v4i none = {-1, -1, -1, -1};
    for (int64_t q = j; q < quads; q += (int64_t)gridDim.x * 256) reinterpret_cast<v4i *>(p.ind_f)[q] = none;
    if (j == 0)
      for (int64_t w = quads << 2; w < words; ++w) p.ind_f[w] = -1;
  }
  if (j < p.n_in && p.mask_b) p.mask_b[j] = 0u;
  if (j >= p.n_out) return;
  Slot *table = reinterpret_cast<Slot *>(p.table);
  unsigned long long key = p.sorted[j];
  uint32_t h = (uint32_t)mix64(key) & p.slot_mask;
  for (uint32_t probe = 0; probe <= p.slot_mask; ++probe) {
    if (table[h].key == key) {
      table[h].row = j;
      break;
    }
    h = (h + 1) & p.slot_mask;
  }
  int4 c;
  c.w = (int)(key % (unsigned long long)p.out_shape[2]); key /= (unsigned long long)p.out_shape[2];
  c.z = (int)(key % (unsigned long long)p.out_shape[1]); key /= (unsigned long long)p.out_shape[1];
  c.y = (int)(key % (unsigned long long)p.out_shape[0]); key /= (unsigned long long)p.out_shape[0];
  c.x = (int)key;
  reinterpret_cast<int4 *>(p.out_coords)[j] = c;
  if (p.mask_f) p.mask_f[j] = 0u;
}

template <bool BITS>
__global__ __launch_bounds__(256) void conv_pairs_fill_kernel(const ConvPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (i >= p.n_in) return;
  unsigned long long key = 0;
  int row = -1;
  if (conv_out_site(p, reinterpret_cast<const int4 *>(p.coords)[i], k, &key)) {
    if constexpr (BITS) {
      const uint32_t word = p.bits[key >> 5], b = (uint32_t)key & 31u;
      if ((word >> b) & 1u) row = (int)(p.prefix[key >> 5] + (uint32_t)__popc(word & ((1u << b) - 1u)));
    } else {
      const Slot *table = reinterpret_cast<const Slot *>(p.table);
      uint32_t h = (uint32_t)mix64(key) & p.slot_mask;
      Slot s = table[h];
      for (uint32_t probe = 0; s.key != key && s.key != kEmptyKey && probe <= p.slot_mask; ++probe) {
        h = (h + 1) & p.slot_mask;
        s = table[h];
      }
      if (s.key == key) row = s.row;
    }
  }
  if (p.ind_b) p.ind_b[(int64_t)k * p.n_in + i] = row;
  if (row >= 0 && row < p.n_out) {
    p.ind_f[(int64_t)k * p.n_out + row] = i;
    if (p.mask_f) atomicOr(&p.mask_f[row], 1u << k);
    if (p.mask_b) atomicOr(&p.mask_b[i], 1u << k);
  }
}

// ---- the same with a bitmap of the output grid in place of the hash set (grids of up to 2^33
// sites): a site's row is the number of set bits before it - a prefix sum over the words' bit
// counts -, so neither the list, nor the sort, nor any probing is needed.
__global__ __launch_bounds__(256) void conv_bits_clear_kernel(const ConvPairsParams p) {
  const v4i zero = {0, 0, 0, 0};   // (n_words is a multiple of 4)
  for (unsigned long long q = blockIdx.x * 256ull + threadIdx.x; q < p.n_words / 4; q += gridDim.x * 256ull)
    reinterpret_cast<v4i *>(p.bits)[q] = zero;
}

__global__ __launch_bounds__(256) void conv_bits_sites_kernel(const ConvPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (i >= p.n_in) return;
  unsigned long long key = 0;
  if (!conv_out_site(p, reinterpret_cast<const int4 *>(p.coords)[i], k, &key)) return;
  const uint32_t bit = 1u << ((uint32_t)key & 31u);
  // a third of the candidates repeat a site: look first (a set bit stays set)
  if (!(__atomic_load_n(&p.bits[key >> 5], __ATOMIC_RELAXED) & bit)) atomicOr(&p.bits[key >> 5], bit);
}

// ---- prefix[w] = number of set bits in the words before w (exclusive scan of the words' bit counts),
// prefix[n_words] = their total.  Three small kernels: bit counts per block of kScanBlock words, one
// workgroup that turns the block counts into offsets (carrying its running sum from one batch of
// 256 blocks to the next), and the scan inside every block again, now with its offset.
constexpr int kScanPerThread = 16;
constexpr int kScanBlock = 256 * kScanPerThread;   // words per workgroup

// a workgroup-wide exclusive scan of one value per thread (256 threads); returns the total in *total
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t *lds_waves, uint32_t *total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t incl = v;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t up = (uint32_t)__shfl_up((int)incl, off, 64);
    if (lane >= off) incl += up;
  }
  __syncthreads();   // (lds_waves may still be read from a previous call)
  if (lane == 63) lds_waves[wave] = incl;
  __syncthreads();
  uint32_t before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const uint32_t c = lds_waves[w];
    before += w < wave ? c : 0u;
    all += c;
  }
  *total = all;
  return before + incl - v;
}

__global__ __launch_bounds__(256) void bit_scan_block_sums_kernel(const uint32_t *__restrict__ bits, unsigned long long n_words,
                                                                  uint32_t *__restrict__ block_sums) {
  __shared__ uint32_t lds_waves[4];
  const unsigned long long base = (unsigned long long)blockIdx.x * kScanBlock;
  uint32_t c = 0;
#pragma unroll
  for (int u = 0; u < kScanPerThread; ++u) {
    const unsigned long long w = base + (unsigned long long)u * 256 + threadIdx.x;
    c += w < n_words ? (uint32_t)__popc(bits[w]) : 0u;
  }
  uint32_t total;
  (void)block_exclusive_scan(c, lds_waves, &total);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

__global__ __launch_bounds__(256) void bit_scan_block_offsets_kernel(uint32_t *__restrict__ block_sums, unsigned long long n_blocks,
                                                                     uint32_t *__restrict__ total_out) {
  __shared__ uint32_t lds_waves[4];
  uint32_t carry = 0;
  for (unsigned long long b0 = 0; b0 < n_blocks; b0 += 256) {
    const unsigned long long b = b0 + threadIdx.x;
    const uint32_t v = b < n_blocks ? block_sums[b] : 0u;
    uint32_t total;
    const uint32_t excl = block_exclusive_scan(v, lds_waves, &total);
    if (b < n_blocks) block_sums[b] = carry + excl;
    carry += total;
  }
  if (threadIdx.x == 0) *total_out = carry;
}

__global__ __launch_bounds__(256) void bit_scan_write_kernel(const uint32_t *__restrict__ bits, unsigned long long n_words,
                                                             const uint32_t *__restrict__ block_sums, uint32_t *__restrict__ prefix) {
  __shared__ uint32_t lds_waves[4];
  // thread t owns kScanPerThread consecutive words (so that its own scan is a running sum)
  const unsigned long long first = (unsigned long long)blockIdx.x * kScanBlock + (unsigned long long)threadIdx.x * kScanPerThread;
  uint32_t cnt[kScanPerThread], mine = 0;
#pragma unroll
  for (int u = 0; u < kScanPerThread; ++u) {
    cnt[u] = first + u < n_words ? (uint32_t)__popc(bits[first + u]) : 0u;
    mine += cnt[u];
  }
  uint32_t total;
  uint32_t run = block_sums[blockIdx.x] + block_exclusive_scan(mine, lds_waves, &total);
#pragma unroll
  for (int u = 0; u < kScanPerThread; ++u) {
    if (first + u < n_words) prefix[first + u] = run;
    run += cnt[u];
  }
}

// ---- the pieces of a 64-bit key sort out of two stable 32-bit sorts (sort_inst.hip)
__global__ __launch_bounds__(256) void key_low_words_kernel(const unsigned long long *__restrict__ keys, uint32_t *__restrict__ out, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (uint32_t)keys[i];
}
__global__ __launch_bounds__(256) void key_high_words_kernel(const unsigned long long *__restrict__ keys, const int32_t *__restrict__ perm,
                                                             uint32_t *__restrict__ out, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (uint32_t)(keys[perm[i]] >> 32);
}
// out[i] = keys[perm1[perm2[i]]] (perm2 NULL: keys[perm1[i]])
__global__ __launch_bounds__(256) void key_gather_kernel(const unsigned long long *__restrict__ keys, const int32_t *__restrict__ perm1,
                                                         const int32_t *__restrict__ perm2, unsigned long long *__restrict__ out, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = keys[perm1[perm2 ? perm2[i] : i]];
}

// table prefill, masks, and the coordinates of the active sites, word by word
__global__ __launch_bounds__(256) void conv_bits_rows_kernel(const ConvPairsParams p) {
  const unsigned long long j = blockIdx.x * 256ull + threadIdx.x, step = gridDim.x * 256ull;
  {
    const unsigned long long words = (unsigned long long)p.kv * p.n_out, quads = words >> 2;
    const v4i none = {-1, -1, -1, -1};
    for (unsigned long long q = j; q < quads; q += step) reinterpret_cast<v4i *>(p.ind_f)[q] = none;
    if (j == 0)
      for (unsigned long long w = quads << 2; w < words; ++w) p.ind_f[w] = -1;
  }
  if (p.mask_b)
    for (unsigned long long i = j; i < (unsigned long long)p.n_in; i += step) p.mask_b[i] = 0u;
  if (p.mask_f)
    for (unsigned long long o = j; o < (unsigned long long)p.n_out; o += step) p.mask_f[o] = 0u;
  for (unsigned long long w = j; w < p.n_words; w += step) {
    uint32_t word = p.bits[w];
    uint32_t row = p.prefix[w];
    while (word != 0u) {
      const int b = __ffs((int)word) - 1;
      word &= word - 1u;
      unsigned long long site = w * 32ull + (unsigned long long)b;
      int4 c;
      c.w = (int)(site % (unsigned long long)p.out_shape[2]); site /= (unsigned long long)p.out_shape[2];
      c.z = (int)(site % (unsigned long long)p.out_shape[1]); site /= (unsigned long long)p.out_shape[1];
      c.y = (int)(site % (unsigned long long)p.out_shape[0]); site /= (unsigned long long)p.out_shape[0];
      c.x = (int)site;
      if (row < (uint32_t)p.n_out) reinterpret_cast<int4 *>(p.out_coords)[row] = c;
      ++row;
    }
  }
}

// ---- per-offset pair lists out of a pair table: what the per-offset ("native") convolution walks
// (spconv's indice_pairs [2, kv, N] and indice_num_per_loc, which the reference's check script
// rebuilds from the mask tables, cumm/conv/main_real_spconv.py:300-326).  Three small kernels:
// pairs per chunk of 2048 entries, an exclusive scan over the chunks of an offset, and the write.
// Within a chunk a thread takes entries t, t + 256, ...: ranks by ballot keep the output rows in
// ascending order.
constexpr int kChunkIters = kPairListChunk / 256;

__global__ __launch_bounds__(256) void pair_lists_count_kernel(const PairListsParams p) {
  __shared__ int wave_cnt[4];
  const int k = blockIdx.y, t = threadIdx.x;
  const int base = blockIdx.x * kPairListChunk;
  int mine = 0;
#pragma unroll
  for (int u = 0; u < kChunkIters; ++u) {
    const int o = base + u * 256 + t;
    const bool have = o < p.n && p.indices[(int64_t)k * p.n + o] >= 0;
    mine += __popcll(__ballot(have));
  }
  if ((t & 63) == 0) wave_cnt[t >> 6] = mine;
  __syncthreads();
  if (t == 0) p.chunk_counts[(int64_t)k * p.chunks + blockIdx.x] = wave_cnt[0] + wave_cnt[1] + wave_cnt[2] + wave_cnt[3];
}

// one workgroup per offset: chunk counts -> exclusive prefix sums (in place), total -> counts[k]
__global__ __launch_bounds__(256) void pair_lists_scan_kernel(const PairListsParams p) {
  __shared__ int lds[256];
  __shared__ int carry;
  const int k = blockIdx.x, t = threadIdx.x;
  int32_t *cc = p.chunk_counts + (int64_t)k * p.chunks;
  if (t == 0) carry = 0;
  __syncthreads();
  for (int c0 = 0; c0 < p.chunks; c0 += 256) {
    const int c = c0 + t;
    const int v = c < p.chunks ? cc[c] : 0;
    lds[t] = v;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      const int add = t >= off ? lds[t - off] : 0;
      __syncthreads();
      lds[t] += add;
      __syncthreads();
    }
    const int base = carry;
    if (c < p.chunks) cc[c] = base + lds[t] - v;
    __syncthreads();
    if (t == 255) carry = base + lds[255];
    __syncthreads();
  }
  if (t == 0) p.counts[k] = carry;
}

__global__ __launch_bounds__(256) void pair_lists_write_kernel(const PairListsParams p) {
  __shared__ int wave_cnt[kChunkIters][4];
  const int k = blockIdx.y, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int base = blockIdx.x * kPairListChunk;
  int in_row[kChunkIters];
  unsigned long long bal[kChunkIters];
#pragma unroll
  for (int u = 0; u < kChunkIters; ++u) {
    const int o = base + u * 256 + t;
    in_row[u] = o < p.n ? p.indices[(int64_t)k * p.n + o] : -1;
    bal[u] = __ballot(in_row[u] >= 0);
    if (lane == 0) wave_cnt[u][wave] = __popcll(bal[u]);
  }
  __syncthreads();
  int at = p.chunk_counts[(int64_t)k * p.chunks + blockIdx.x];
#pragma unroll
  for (int u = 0; u < kChunkIters; ++u) {
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int c = wave_cnt[u][w];
      before += w < wave ? c : 0;
      total += c;
    }
    if (in_row[u] >= 0) {
      const int64_t dst = (int64_t)k * p.n + at + before + __popcll(bal[u] & ((1ull << lane) - 1ull));
      p.pair_in[dst] = in_row[u];
      p.pair_out[dst] = base + u * 256 + t;
    }
    at += total;
  }
}

// mask[o * words + w] = bit b set wherever indices[32 w + b][o] >= 0: the masks of a pair table,
// any kernel volume (one lane per output, walking the offsets: every table row is read coalesced)
__global__ __launch_bounds__(256) void masks_from_pairs_kernel(const int32_t *__restrict__ indices, uint32_t *__restrict__ mask,
                                                               int kv, int n, int words) {
  const int o = blockIdx.x * 256 + threadIdx.x;
  if (o >= n) return;
  for (int w = 0; w < words; ++w) {
    uint32_t m = 0;
    const int hi = kv - 32 * w < 32 ? kv - 32 * w : 32;
    for (int b = 0; b < hi; ++b) m |= indices[(int64_t)(32 * w + b) * n + o] >= 0 ? 1u << b : 0u;
    mask[(int64_t)o * words + w] = m;
  }
}

// Sort key of a position with several mask words: positions with few offsets first (the number
// of offsets in the upper six bits, at most 63), equal masks next to each other (a 26-bit hash of
// the words below it).  Any order is a valid input of the convolution kernels; this one makes the
// tiles of the light end light.
__device__ __forceinline__ uint32_t mask_words_key(const uint32_t *w, int words) {
  uint32_t pc = 0, h = 0;
  for (int i = 0; i < words; ++i) {
    pc += (uint32_t)__builtin_popcount(w[i]);
    const int r = (7 * i) & 31;
    h ^= r ? (w[i] << r) | (w[i] >> (32 - r)) : w[i];
  }
  return ((pc < 63u ? pc : 63u) << 26) | ((h * 0x9E3779B1u) >> 6);
}
__global__ __launch_bounds__(256) void mask_words_keys_kernel(const uint32_t *__restrict__ mask, uint32_t *__restrict__ keys,
                                                              int n, int words) {
  const int o = blockIdx.x * 256 + threadIdx.x;
  if (o >= n) return;
  uint32_t w[4] = {0u, 0u, 0u, 0u};
  for (int i = 0; i < words && i < 4; ++i) w[i] = mask[(int64_t)o * words + i];
  keys[o] = mask_words_key(w, words < 4 ? words : 4);
}
__global__ __launch_bounds__(256) void mask_words_gather_kernel(const uint32_t *__restrict__ mask, const int32_t *__restrict__ argsort,
                                                                uint32_t *__restrict__ sorted, int n, int words) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (int64_t)n * words) return;
  const int pos = (int)(i / words), w = (int)(i % words);
  const int row = argsort[pos];
  sorted[i] = row >= 0 && row < n ? mask[(int64_t)row * words + w] : 0u;
}

// out[k][pos] = indices[k][argsort[pos]]: the pair table in the order of the sorted positions
__global__ __launch_bounds__(256) void pairs_by_position_kernel(const int32_t *__restrict__ indices,
                                                                const int32_t *__restrict__ argsort,
                                                                int32_t *__restrict__ out, int n, int rows) {
  const int pos = blockIdx.x * 256 + threadIdx.x;
  if (pos >= n) return;
  const int row = argsort[pos];
  const int64_t k = blockIdx.y;
  out[k * n + pos] = row >= 0 && row < rows ? indices[k * rows + row] : -1;
}

}  // namespace

hipError_t launch_masks_from_pairs(const int32_t *indices, uint32_t *mask, int kv, int n, hipStream_t s) {
  if (kv <= 0 || n <= 0) return hipSuccess;
  hipLaunchKernelGGL(masks_from_pairs_kernel, dim3((n + 255) / 256), dim3(256), 0, s, indices, mask, kv, n, (kv + 31) / 32);
  return hipGetLastError();
}
hipError_t launch_mask_words_keys(const uint32_t *mask, uint32_t *keys, int n, int words, hipStream_t s) {
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(mask_words_keys_kernel, dim3((n + 255) / 256), dim3(256), 0, s, mask, keys, n, words);
  return hipGetLastError();
}
hipError_t launch_mask_words_gather(const uint32_t *mask, const int32_t *argsort, uint32_t *sorted, int n, int words, hipStream_t s) {
  if (n <= 0) return hipSuccess;
  const int64_t total = (int64_t)n * words;
  hipLaunchKernelGGL(mask_words_gather_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, mask, argsort, sorted, n, words);
  return hipGetLastError();
}

hipError_t launch_pairs_by_position(const int32_t *indices, const int32_t *argsort, int32_t *out, int kv, int n, int rows,
                                    hipStream_t s) {
  if (kv <= 0 || n <= 0) return hipSuccess;
  hipLaunchKernelGGL(pairs_by_position_kernel, dim3((n + 255) / 256, kv), dim3(256), 0, s, indices, argsort, out, n, rows);
  return hipGetLastError();
}

hipError_t launch_pair_lists(const PairListsParams &p, hipStream_t s) {
  if (p.kv <= 0) return hipSuccess;
  if (p.n <= 0 || p.chunks <= 0) {
    hipLaunchKernelGGL(pair_lists_scan_kernel, dim3(p.kv), dim3(256), 0, s, p);   // (counts = 0)
    return hipGetLastError();
  }
  hipLaunchKernelGGL(pair_lists_count_kernel, dim3(p.chunks, p.kv), dim3(256), 0, s, p);
  hipLaunchKernelGGL(pair_lists_scan_kernel, dim3(p.kv), dim3(256), 0, s, p);
  hipLaunchKernelGGL(pair_lists_write_kernel, dim3(p.chunks, p.kv), dim3(256), 0, s, p);
  return hipGetLastError();
}

hipError_t launch_conv_pairs_sites(const ConvPairsParams &p, hipStream_t s) {
  hipLaunchKernelGGL(conv_pairs_clear_kernel, dim3((p.slot_mask + 256u) / 256u), dim3(256), 0, s, p);
  if (p.n_in > 0) {
    hipLaunchKernelGGL(conv_pairs_sites_kernel, dim3((p.n_in + 255) / 256, p.kv), dim3(256), 0, s, p);
    const uint32_t per_wg = 256u * kCompactPerThread;
    hipLaunchKernelGGL(conv_pairs_compact_kernel, dim3((p.slot_mask + per_wg) / per_wg), dim3(256), 0, s, p);
  }
  return hipGetLastError();
}

// 64-bit keys, ascending: a stable sort by the low words, then a stable sort of that order by the
// high words (skipped when no key has any), each the radix sort of the mask sort.
// temp: six arrays of n words (low words, their sorted copy, the first order, high words in that
// order, their sorted copy, the second order) and the sort's own workspace.
static size_t key_sort_part(size_t n) { return (4 * (n > 0 ? n : 1) + 255) & ~(size_t)255; }
size_t conv_pairs_sort_temp_bytes(size_t max_sites) {
  return 6 * key_sort_part(max_sites) + sort_by_mask_workspace_bytes((int)(max_sites > 0 ? max_sites : 1));
}

hipError_t launch_conv_pairs_sort(const ConvPairsParams &p, unsigned long long max_key, void *temp, size_t temp_bytes,
                                  int32_t *give_ups, hipStream_t s) {
  if (p.n_out <= 0) return hipSuccess;
  const int n = p.n_out;
  if (temp_bytes < conv_pairs_sort_temp_bytes((size_t)n)) return hipErrorInvalidValue;
  const size_t part = key_sort_part((size_t)n);
  char *base = reinterpret_cast<char *>(temp);
  uint32_t *lo = reinterpret_cast<uint32_t *>(base), *lo_sorted = reinterpret_cast<uint32_t *>(base + part);
  int32_t *perm1 = reinterpret_cast<int32_t *>(base + 2 * part);
  uint32_t *hi = reinterpret_cast<uint32_t *>(base + 3 * part), *hi_sorted = reinterpret_cast<uint32_t *>(base + 4 * part);
  int32_t *perm2 = reinterpret_cast<int32_t *>(base + 5 * part);
  void *sort_ws = base + 6 * part;
  const dim3 grid((n + 255) / 256);
  hipLaunchKernelGGL(key_low_words_kernel, grid, dim3(256), 0, s, p.uniq, lo, n);
  hipError_t e = launch_sort_by_mask(lo, n, 0xFFFFFFFFu, lo_sorted, perm1, sort_ws, give_ups, nullptr, 0, s);
  if (e != hipSuccess) return e;
  const bool two = (max_key >> 32) != 0ull;
  if (two) {
    hipLaunchKernelGGL(key_high_words_kernel, grid, dim3(256), 0, s, p.uniq, perm1, hi, n);
    uint32_t filter = 1;
    while (filter != 0xFFFFFFFFu && (max_key >> 32) > filter) filter = (filter << 1) | 1u;   // the bits the high words use
    e = launch_sort_by_mask(hi, n, filter, hi_sorted, perm2, sort_ws, give_ups, nullptr, 0, s);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(key_gather_kernel, grid, dim3(256), 0, s, p.uniq, perm1, two ? perm2 : nullptr, p.sorted, n);
  return hipGetLastError();
}

hipError_t launch_conv_pairs_fill(const ConvPairsParams &p, hipStream_t s) {
  const int most = p.n_out > p.n_in ? p.n_out : p.n_in;
  if (most <= 0) return hipSuccess;
  if (p.n_words != 0ull) {
    unsigned long long wgs = (p.n_words + 255ull) / 256ull;
    if (wgs < (unsigned long long)(most + 255) / 256) wgs = (unsigned long long)(most + 255) / 256;
    if (wgs > 16384ull) wgs = 16384ull;
    hipLaunchKernelGGL(conv_bits_rows_kernel, dim3((unsigned)wgs), dim3(256), 0, s, p);
    if (p.n_in > 0)
      hipLaunchKernelGGL(conv_pairs_fill_kernel<true>, dim3((p.n_in + 255) / 256, p.kv), dim3(256), 0, s, p);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(conv_pairs_rows_kernel, dim3((most + 255) / 256), dim3(256), 0, s, p);
  if (p.n_in > 0)
    hipLaunchKernelGGL(conv_pairs_fill_kernel<false>, dim3((p.n_in + 255) / 256, p.kv), dim3(256), 0, s, p);
  return hipGetLastError();
}

// block counts of the bit scan
size_t conv_pairs_scan_temp_bytes(size_t n_words) {
  return 4 * ((n_words + kScanBlock - 1) / kScanBlock + 1);
}

// bitmap of the active output sites and its prefix sums
hipError_t launch_conv_pairs_bits(const ConvPairsParams &p, void *temp, size_t temp_bytes, hipStream_t s) {
  unsigned long long wgs = (p.n_words / 4 + 255ull) / 256ull;
  if (wgs > 16384ull) wgs = 16384ull;
  if (wgs == 0ull) wgs = 1ull;
  hipLaunchKernelGGL(conv_bits_clear_kernel, dim3((unsigned)wgs), dim3(256), 0, s, p);
  if (p.n_in > 0)
    hipLaunchKernelGGL(conv_bits_sites_kernel, dim3((p.n_in + 255) / 256, p.kv), dim3(256), 0, s, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const unsigned long long n_blocks = (p.n_words + kScanBlock - 1) / kScanBlock;
  if (n_blocks == 0ull || n_blocks > 0x7fffffffull || temp_bytes < conv_pairs_scan_temp_bytes((size_t)p.n_words)) return hipErrorInvalidValue;
  uint32_t *block_sums = reinterpret_cast<uint32_t *>(temp);
  hipLaunchKernelGGL(bit_scan_block_sums_kernel, dim3((unsigned)n_blocks), dim3(256), 0, s, p.bits, p.n_words, block_sums);
  hipLaunchKernelGGL(bit_scan_block_offsets_kernel, dim3(1), dim3(256), 0, s, block_sums, n_blocks, p.prefix + p.n_words);
  hipLaunchKernelGGL(bit_scan_write_kernel, dim3((unsigned)n_blocks), dim3(256), 0, s, p.bits, p.n_words, block_sums, p.prefix);
  return hipGetLastError();
}

hipError_t launch_subm_pairs(const SubmPairsParams &p, hipStream_t s) {
  if (p.n <= 0) return hipSuccess;
  uint32_t most = p.slot_mask + 1u;   // (>= 2 n and >= the presence words)
  if (p.filter_mask + 1u > most) most = p.filter_mask + 1u;
  if ((uint32_t)p.n > most) most = (uint32_t)p.n;
  hipLaunchKernelGGL(pairs_clear_kernel, dim3((most + 255) / 256), dim3(256), 0, s, p);
  hipLaunchKernelGGL(pairs_insert_kernel, dim3((p.n + 255) / 256), dim3(256), 0, s, p);
  hipLaunchKernelGGL(pairs_lookup_kernel, dim3((p.n + 255) / 256, p.kv / p.kx), dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace cummhip
