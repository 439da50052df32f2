// Host-side launch tables: one function per element type, defined in its own translation unit so
// that the kernel instantiations compile in parallel.
#pragma once
#include "rowgemm.h"
#include "tilegemm.h"
#include "wgrad_atomic.h"

namespace cummhip {

// The kernels that count their vector-memory loads by hand (direct-to-LDS loads and register
// loads issued from asm statements, waited for with s_waitcnt vmcnt(n)) are correct only while
// the compiler adds no vector-memory access of its own between a load and its wait: a register
// spilled to scratch memory is one (scratch accesses count in vmcnt like any other).  Checked
// once per kernel, when it is first launched, on the code object that was actually loaded: a
// kernel with private (scratch) memory is not launched; the caller falls back to a kernel without
// counted waits or reports the launch as failed.
template <auto Kernel>
inline bool counted_waits_hold() {
  static const bool ok = [] {
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(Kernel)) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    return attr.localSizeBytes == 0;
  }();
  return ok;
}

// returns hipSuccess, or hipErrorInvalidValue when no instantiation matches
hipError_t launch_rowgemm_f16(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);
hipError_t launch_rowgemm_bf16(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);
hipError_t launch_rowgemm_s8(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);

// the same tables with four-byte outputs (s32 for s8 operands, f32 for f16 / bf16)
hipError_t launch_rowgemm_wide_f16(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);
hipError_t launch_rowgemm_wide_bf16(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);
hipError_t launch_rowgemm_wide_s8(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);

hipError_t launch_tilegemm_f16(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                               hipStream_t s);
hipError_t launch_tilegemm_bf16(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                                hipStream_t s);
hipError_t launch_tilegemm_s8(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                              hipStream_t s);

hipError_t launch_tilegemm_wide_f16(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                                    hipStream_t s);
hipError_t launch_tilegemm_wide_bf16(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                                     hipStream_t s);
hipError_t launch_tilegemm_wide_s8(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                                   hipStream_t s);

// balanced backward-weight with fp32 atomics: main kernel then finalize (f16 / bf16 only)
hipError_t launch_wgrad_atomic_f16(const WgradParams &p, const WgradPrepareParams &pre, const WgradFinalizeParams &f, hipStream_t s);
hipError_t launch_wgrad_atomic_bf16(const WgradParams &p, const WgradPrepareParams &pre, const WgradFinalizeParams &f, hipStream_t s);
int wgrad_ordered_resident_f16(bool wide);
int wgrad_ordered_resident_bf16(bool wide);
hipError_t launch_wgrad_ordered_f16(const WgradParams &p, const WgradPrepareParams &pre, const WgradOrderedParams &f, bool wide, int wgs, hipStream_t s);
hipError_t launch_wgrad_ordered_bf16(const WgradParams &p, const WgradPrepareParams &pre, const WgradOrderedParams &f, bool wide, int wgs, hipStream_t s);

// tile shapes the tables above hold
inline bool rowgemm_has_tile(int tm, int tn) {
  return (tm == 64 || tm == 128) && (tn == 64 || tn == 128);
}
inline bool tilegemm_has_tile(int tm, int tn) {
  return (tm == 64 && tn == 64) || (tm == 128 && tn == 128);
}

// Largest kernel volume the pair builders take (5 x 5 x 5).  Volumes above 32 have no 32-bit
// masks: their tables feed the per-offset ("native") convolution, not the mask-based kernels.
constexpr int kMaxKernelVolume = 128;

// ---- pair tables of a submanifold convolution and the mask sort (pairs_inst.hip)
struct SubmPairsParams {
  const int32_t *coords;   // [n, 4] (batch, z, y, x)
  int32_t n, kv;
  int32_t shape[3];
  int32_t off[kMaxKernelVolume][3];   // (k_zyx - center) * dilation per kernel offset
  int32_t *ind_f, *ind_b;  // [kv, n]; ind_b may be NULL
  uint32_t *mask_f, *mask_b;   // may be NULL (must be for kernel volumes above 32)
  void *table;             // (slot_mask + 1) slots of 16 bytes
  uint32_t slot_mask;
  uint32_t *filter;        // (filter_mask + 1) presence words
  uint32_t filter_mask;
  int32_t kx;              // offsets along x (kv = kz * ky * kx)
  int32_t center_k;        // the offset (0, 0, 0), whose pair is the voxel itself; -1 if there is none
};
hipError_t launch_subm_pairs(const SubmPairsParams &p, hipStream_t s);

// ---- pair tables of a regular (strided) sparse convolution (pairs_inst.hip)
struct ConvPairsParams {
  const int32_t *coords;        // [n_in, 4] (batch, z, y, x)
  int32_t n_in, n_out, kv, batch;
  int32_t out_shape[3], stride[3], pad[3];
  int32_t koff[kMaxKernelVolume][3];   // k_zyx * dilation per kernel offset
  void *table;                  // (slot_mask + 1) slots of 16 bytes: {output site key, output row}
  uint32_t slot_mask;
  unsigned long long *uniq;     // output site keys in order of discovery
  unsigned long long *sorted;   // the same, ascending = output rows
  unsigned long long *counters; // [0] number of output sites, [1] largest key
  uint32_t *bits;               // instead of the table, for a small output grid: one bit per site,
  uint32_t *prefix;             // and the number of active sites before each 32-bit word
  unsigned long long n_words;   // (0 = hash set and sort)
  int32_t *out_coords;          // [n_out, 4]
  int32_t *ind_f, *ind_b;       // [kv, n_out], [kv, n_in] (may be NULL)
  uint32_t *mask_f, *mask_b;    // [n_out], [n_in] (may be NULL; must be for kernel volumes above 32)
};
hipError_t launch_conv_pairs_sites(const ConvPairsParams &p, hipStream_t s);
size_t conv_pairs_sort_temp_bytes(size_t max_sites);
hipError_t launch_conv_pairs_sort(const ConvPairsParams &p, unsigned long long max_key, void *temp, size_t temp_bytes,
                                  int32_t *give_ups, hipStream_t s);
hipError_t launch_conv_pairs_fill(const ConvPairsParams &p, hipStream_t s);
size_t conv_pairs_scan_temp_bytes(size_t n_words);
hipError_t launch_conv_pairs_bits(const ConvPairsParams &p, void *temp, size_t temp_bytes, hipStream_t s);
// What input preparation knows about a sorted mask array and a later forward / backward-input
// launch on the same array can use without being told: a table of kLightHintSlots slots of eight
// words in device memory, one table per GPU, indexed by a hash of the array's address.  Slot =
// {address (two words), length, filter, light prefix in positions, first position of the heavy
// end (the length rounded up to 64 = none), 1 if sorted by offset count, 0}.  A hint only: a
// launch that finds another array's slot, or a stale one, or none, still computes the same bits.
constexpr int kLightHintSlots = 256;
inline int light_hint_slot(const void *sorted_mask) {
  const uint64_t a = reinterpret_cast<uintptr_t>(sorted_mask) >> 8;
  return (int)(((a * 0x9E3779B97F4A7C15ull) >> 40) & (uint64_t)(kLightHintSlots - 1));
}
// stable radix sort of mask & filter with its permutation (sort_inst.hip)
size_t sort_by_mask_workspace_bytes(int n);
// light prefix of a sorted array into *result (may be NULL) and into hint_slot (may be NULL)
hipError_t launch_light_prefix(const uint32_t *sorted, int n, uint32_t filter, int32_t *result, int32_t *hint_slot,
                               hipStream_t s);
// hint_slot: the slot of `sorted` in the current device's table (NULL = leave no hint)
// order 0: ascending mask value; 1: ascending number of offsets, then value (filter below 2^27)
hipError_t launch_sort_by_mask(const uint32_t *mask, int n, uint32_t filter, uint32_t *sorted, int32_t *argsort,
                               void *workspace, int32_t *give_ups, int32_t *hint_slot, int order, hipStream_t s);

// per-offset lists of (input row, output row) out of a pair table [kv, n] (pairs_inst.hip)
struct PairListsParams {
  const int32_t *indices;   // [kv, n]: input row of output o at offset k, -1 = none
  int32_t *pair_in, *pair_out;   // [kv, n] each: the pairs of offset k, ascending output row, packed to the front
  int32_t *counts;          // [kv]
  int32_t *chunk_counts;    // [kv, chunks] scratch
  int32_t kv, n, chunks;
};
hipError_t launch_masks_from_pairs(const int32_t *indices, uint32_t *mask, int kv, int n, hipStream_t s);
hipError_t launch_mask_words_keys(const uint32_t *mask, uint32_t *keys, int n, int words, hipStream_t s);
hipError_t launch_mask_words_gather(const uint32_t *mask, const int32_t *argsort, uint32_t *sorted, int n, int words, hipStream_t s);
hipError_t launch_pairs_by_position(const int32_t *indices, const int32_t *argsort, int32_t *out, int kv, int n, int rows,
                                    hipStream_t s);
constexpr int kPairListChunk = 2048;   // table entries per workgroup
hipError_t launch_pair_lists(const PairListsParams &p, hipStream_t s);

// ---- stand-alone row gather / scatter-add (gather_inst.hip)
struct RowMoveParams {
  const void *src;
  void *dst;
  const int32_t *indices;   // [m]
  uint64_t pieces;          // m * per_row
  uint32_t per_row;         // pieces (16 or 4 bytes) per row
  int32_t shift;            // log2(per_row) when that is a power of two, else -1
  int32_t rows_other;       // rows of the indexed tensor (gather: source, scatter-add: destination)
};
hipError_t launch_gather_rows(const RowMoveParams &p, bool wide, hipStream_t s);
hipError_t launch_scatter_add_rows(const RowMoveParams &p, int dtype, bool wide, hipStream_t s);

// ---- row-wise helpers (elementwise_inst.hip)
struct FinishRowsParams {
  void *out;            // [rows, channels] f16 / bf16
  const float *acc;     // [rows, channels] fp32
  const void *bias;     // [channels] in the output's type, or NULL
  int64_t rows;
  int32_t channels;     // a multiple of 8
  float alpha, beta, act_alpha;
  int32_t act;
};
hipError_t launch_finish_rows(const FinishRowsParams &p, bool bf16, hipStream_t s);
hipError_t launch_relu_backward(void *dst, const void *grad, const void *out, size_t vecs, bool bf16, hipStream_t s);
struct ColumnSumParams {
  void *dst;            // [channels]
  const void *src;      // [rows, channels]
  float *partial;       // [blocks, channels] fp32
  int64_t rows, rows_per_block;
  int32_t channels, blocks;
};
int column_sum_blocks(int64_t rows, int channels);
hipError_t launch_column_sum(ColumnSumParams p, bool bf16, hipStream_t s);

}  // namespace cummhip
