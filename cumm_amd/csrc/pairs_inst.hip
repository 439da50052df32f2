// Pair tables of a submanifold convolution and the mask sort, on the GPU: the step right before
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
//   * the mask sort is rocPRIM's radix sort by key (stable, like the host's argsort).
#include <hip/hip_runtime.h>

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

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
    p.mask_f[i] = 0u;
    if (p.mask_b) p.mask_b[i] = 0u;
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
      atomicOr(&p.mask_f[i], 1u << k);
      if (p.mask_b) atomicOr(&p.mask_b[i], 1u << (p.kv - 1 - k));
    }
  }
}

__global__ __launch_bounds__(256) void sort_keys_kernel(const uint32_t *mask, uint32_t filter, uint32_t *keys,
                                                        int32_t *iota, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  keys[i] = mask[i] & filter;
  iota[i] = i;
}

}  // namespace

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

size_t sort_by_mask_temp_bytes(int n) {
  size_t bytes = 0;
  (void)rocprim::radix_sort_pairs(nullptr, bytes, (const uint32_t *)nullptr, (uint32_t *)nullptr, (const int32_t *)nullptr,
                            (int32_t *)nullptr, (size_t)(n > 0 ? n : 1), 0, 32);
  return bytes;
}

hipError_t launch_sort_by_mask(const uint32_t *mask, int n, uint32_t filter, uint32_t *sorted, int32_t *argsort,
                               void *keys_ws, void *iota_ws, void *temp, size_t temp_bytes, hipStream_t s) {
  // only the bits the filter lets through can differ: fewer radix passes
  int end_bit = 32;
  while (end_bit > 1 && !((filter >> (end_bit - 1)) & 1u)) --end_bit;
  if (n <= 0) return hipSuccess;
  hipLaunchKernelGGL(sort_keys_kernel, dim3((n + 255) / 256), dim3(256), 0, s, mask, filter,
                     reinterpret_cast<uint32_t *>(keys_ws), reinterpret_cast<int32_t *>(iota_ws), n);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  return rocprim::radix_sort_pairs(temp, temp_bytes, reinterpret_cast<const uint32_t *>(keys_ws), sorted,
                                   reinterpret_cast<const int32_t *>(iota_ws), argsort, (size_t)n, 0, end_bit, s);
}

}  // namespace cummhip
