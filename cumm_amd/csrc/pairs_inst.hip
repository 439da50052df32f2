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
//   * the lookup kernel is one lane per (voxel, offset): for a fixed offset consecutive lanes
//     write consecutive table entries (coalesced), and kv times more lanes than voxels hide the
//     probe latency (one lane per voxel walking its 27 offsets took 127 us for 120 k voxels);
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

__global__ __launch_bounds__(256) void pairs_clear_kernel(Slot *table, uint32_t slots) {
  const uint32_t i = blockIdx.x * 256u + threadIdx.x;
  if (i < slots) table[i] = Slot{kEmptyKey, -1, 0};
}

__device__ __forceinline__ unsigned long long coord_key(int b, int z, int y, int x, const SubmPairsParams &p) {
  return (((unsigned long long)b * p.shape[0] + z) * p.shape[1] + y) * p.shape[2] + x;
}

__global__ __launch_bounds__(256) void pairs_insert_kernel(const SubmPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= p.n) return;
  const int4 c = reinterpret_cast<const int4 *>(p.coords)[i];
  const unsigned long long key = coord_key(c.x, c.y, c.z, c.w, p);
  Slot *table = reinterpret_cast<Slot *>(p.table);
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

// One lane per (voxel, kernel offset): grid.y = kernel offsets, consecutive lanes = consecutive
// voxels, so both table rows are written coalesced; 27 times more lanes than voxels hide the
// probe latency.  The masks are OR-ed with atomics, one per PAIR (1.5 per voxel on the benchmark
// cloud), into words that the clear kernel zeroed.
__global__ __launch_bounds__(256) void pairs_lookup_kernel(const SubmPairsParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (i >= p.n) return;
  const int4 c = reinterpret_cast<const int4 *>(p.coords)[i];
  const Slot *table = reinterpret_cast<const Slot *>(p.table);
  const int z = c.y + p.off[k][0], y = c.z + p.off[k][1], x = c.w + p.off[k][2];
  int row = -1;
  if (z >= 0 && z < p.shape[0] && y >= 0 && y < p.shape[1] && x >= 0 && x < p.shape[2]) {
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
  p.ind_f[(int64_t)k * p.n + i] = row;
  if (p.ind_b) p.ind_b[(int64_t)(p.kv - 1 - k) * p.n + i] = row;
  if (row >= 0) {
    atomicOr(&p.mask_f[i], 1u << k);
    if (p.mask_b) atomicOr(&p.mask_b[i], 1u << (p.kv - 1 - k));
  }
}

__global__ __launch_bounds__(256) void pairs_zero_masks_kernel(uint32_t *mask_f, uint32_t *mask_b, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  mask_f[i] = 0u;
  if (mask_b) mask_b[i] = 0u;
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
  const uint32_t slots = p.slot_mask + 1u;
  hipLaunchKernelGGL(pairs_clear_kernel, dim3((slots + 255) / 256), dim3(256), 0, s, reinterpret_cast<Slot *>(p.table), slots);
  hipLaunchKernelGGL(pairs_zero_masks_kernel, dim3((p.n + 255) / 256), dim3(256), 0, s, p.mask_f, p.mask_b, p.n);
  hipLaunchKernelGGL(pairs_insert_kernel, dim3((p.n + 255) / 256), dim3(256), 0, s, p);
  hipLaunchKernelGGL(pairs_lookup_kernel, dim3((p.n + 255) / 256, p.kv), dim3(256), 0, s, p);
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
