/*
 * cumm_hip.h - C ABI of libcummhip.so: gfx950 (MI355X) kernels for the GEMM and
 * mask-based implicit-GEMM sparse-convolution path of FindDefinition/cumm.
 *
 * Every entry point takes plain pointers and sizes (device pointers unless a
 * comment says host) and returns 0 on success or a CUMM_HIP_E* code; the text
 * of the last error of the calling thread is read with cumm_hip_last_error().
 * Launches are asynchronous on the given stream (0 = the default stream); no
 * entry point synchronises unless its name says so.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the reference tree).
 */
#ifndef CUMM_HIP_H_
#define CUMM_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* status codes */
#define CUMM_HIP_OK 0
#define CUMM_HIP_EINVAL 1      /* bad argument: the reference raises ValueError (TV_ASSERT_INVALID_ARG) */
#define CUMM_HIP_ERUNTIME 2    /* failed check / HIP error: the reference raises RuntimeError (TV_ASSERT_RT_ERR) */
#define CUMM_HIP_ENOALGO 3     /* no kernel for this descriptor ("can't find any suitable algo") */

/* tv::DType values, include/tensorview/dtypes.h:39-64 */
#define CUMM_HIP_F32 0
#define CUMM_HIP_S32 1
#define CUMM_HIP_S8 3
#define CUMM_HIP_F16 7
#define CUMM_HIP_U32 10
#define CUMM_HIP_BF16 12

/* tv::gemm::ConvOpType / ShuffleStrideType / Activation,
 * include/tensorview/gemm/core/constants.h:20-55 */
#define CUMM_HIP_OP_FORWARD 0
#define CUMM_HIP_OP_BACKWARD_INPUT 1
#define CUMM_HIP_OP_BACKWARD_WEIGHT 2
#define CUMM_HIP_NO_SHUFFLE 0
#define CUMM_HIP_SHUFFLE_AC 1
#define CUMM_HIP_SHUFFLE_AB 2
#define CUMM_HIP_CONV_CONVOLUTION 0
#define CUMM_HIP_CONV_CROSS_CORRELATION 1
#define CUMM_HIP_ACT_NONE 0
#define CUMM_HIP_ACT_RELU 1
#define CUMM_HIP_ACT_SIGMOID 2
#define CUMM_HIP_ACT_LEAKY_RELU 3

/* The fields of tv::gemm::GemmAlgoDesp that select a kernel
 * (include/tensorview/gemm/core/params.h:24-54).  num_stage is 2 except for the second descriptor of
 * the 128 x 128 forward / backward-input tile (f16, bf16), where 3 selects three small stages for
 * contractions of more than 128 bytes per row: same results to the bit, faster where tiles have
 * few kernel offsets, slower where they have many - a choice for the caller's tuner. */
typedef struct CummHipGemmDesc {
  int32_t dtype_a, dtype_b, dtype_c, dacc, dcomp;
  int32_t trans_a, trans_b, trans_c;
  int32_t tile_shape[3];
  int32_t warp_tile_shape[3];
  int32_t num_stage;
  int32_t shuffle_type;
  int32_t split_k_serial, split_k_parallel;
} CummHipGemmDesc;

/* tv::gemm::ConvAlgoDesp adds these (params.h:166-196). */
typedef struct CummHipConvDesc {
  CummHipGemmDesc gemm;
  int32_t ndim, op_type;
  int32_t mask_sparse, increment_k_first, dynamic_mask, is_int8_inference;
} CummHipConvDesc;

/* Operands of one GEMM launch: tv::gemm::GemmNVRTCParams
 * (include/tensorview/gemm/core/nvrtc_params.h:23-37) as filled by the prelude
 * cumm/gemm/nvrtc_code.py:34-198.  Strides are row strides in elements;
 * stride_D == 0 means D is a bias over n. */
typedef struct CummHipGemmArgs {
  int32_t m, n, k;
  const void *ptr_A, *ptr_B, *ptr_D;
  void *ptr_C;
  int64_t stride_A, stride_B, stride_C, stride_D;
  const int32_t *indiceA;    /* ShuffleAC: a_inds or NULL; ShuffleAB: a_inds */
  const int32_t *indiceBorC; /* ShuffleAC: c_inds; ShuffleAB: b_inds */
  const int32_t *indiceD;    /* ShuffleAC: c_inds or NULL when D is a bias */
  float alpha, beta, act_alpha, act_beta;
  int32_t act_type;
  int32_t split_k_slices;
  void *workspace;           /* split-K scratch, zeroed by the callee before use */
  size_t workspace_bytes;
  int32_t rows_A, rows_B, rows_C; /* row counts of the underlying tensors: gathered/scattered
                                     row numbers outside them are treated as absent */
} CummHipGemmArgs;

/* Operands of one mask-based sparse-convolution launch:
 * tv::gemm::SparseConvNVRTCParams (nvrtc_params.h:39-65) as filled by the
 * prelude cumm/conv/nvrtc_code.py:20-197.  (A,B,C) are (input,weight,output)
 * permuted by op_type exactly as there: forward (input, weight, output),
 * dgrad (output, weight, input), wgrad (output, input, weight).
 * Rows of input/output are dense (row stride == channel count); the weight is
 * [K, kernel_volume, C]. */
typedef struct CummHipSparseConvArgs {
  const void *ptr_A, *ptr_B, *ptr_D;
  void *ptr_C;
  float alpha, beta, act_alpha, act_beta;
  int32_t act_type;
  int32_t split_k_slices;
  void *workspace;
  size_t workspace_bytes;
  const uint32_t *mask_ptr;         /* fwd/dgrad: per sorted position; wgrad: forward's mask_output */
  uint32_t *mask_out_ptr;           /* forward only, may be NULL */
  const int32_t *indice_ptr;        /* [kernel_volume, N] */
  const int32_t *mask_argsort_ptr;  /* [N] */
  uint32_t mask_filter;
  int32_t reverse_mask;
  int32_t mask_width;               /* wgrad: positions covered by one mask word */
  int32_t ndim, N, C, K;
  int32_t kernel_volume;
  int32_t mode;                     /* tv::gemm::ConvMode: must be CUMM_HIP_CONV_CROSS_CORRELATION, the only one
                                       the reference's mask-based kernels implement */
  int32_t groups;                   /* must be 1 */
  int32_t d_is_bias;
  int32_t deterministic;            /* backward-weight with a split_k_parallel descriptor: non-zero = partial sums
                                       added in a fixed order (same bits from run to run on one device), as the
                                       reference's serial split-K is (cumm/conv/kernel.py:1004-1014, 1068-1083);
                                       workspace: cumm_hip_query_wgrad_ordered_workspace.  Ignored elsewhere. */
  const void *bias_pointer;         /* int8 inference: f32 [K] */
  const void *scale_pointer;        /* int8 inference: f32 [K] */
  int32_t rows_in, rows_out;        /* row counts of the input / output feature tensors */
  int32_t light_prefix;             /* forward / backward-input, optional: how many leading positions of the sorted order
                                       sit in tiles of one or two kernel offsets, as cumm_hip_light_prefix counts them
                                       for mask_ptr.  A hint only: it moves those positions to 128-row tiles (fewer,
                                       longer-lived workgroups where a tile's time is its memory round trips); any
                                       value gives the same bits, a wrong one costs time.  0 (what a caller that fills
                                       the reference's struct passes) = not given: the launch then uses the count that
                                       cumm_hip_sort_by_mask or cumm_hip_light_prefix left for this mask array in the
                                       library's own table on the device, if there is one.  Negative = no hint at all.
                                       No counterpart in the reference. */
  int32_t ungated_rows;             /* forward / backward-input.  0: a position takes part in kernel offset k only if its
                                       own mask word has bit k - masks made from the pair table (bit k set wherever
                                       indice_ptr[k][row] >= 0, as spconv makes them) lose nothing, and entries and rows
                                       of the other offsets are never fetched.  Non-zero: every position of a tile takes
                                       part in every offset of the tile's OR-ed mask and is gated by its pair-table entry
                                       alone - the reference's rule (cumm/conv/sparse_iters.py:629-631), which differs
                                       from the above only for masks with a bit clear over a valid entry; slower
                                       (the hint light_prefix is then ignored). */
  int32_t indices_by_position;      /* forward / backward-input.  Non-zero: indice_ptr is the pair table in the order of
                                       the sorted positions, [kernel_volume, N] with entry [k][pos] = the reference
                                       table's [k][mask_argsort_ptr[pos]] (cumm_hip_pairs_by_position makes it, once per
                                       geometry and sort).  A tile's entries for one offset are then consecutive in
                                       memory instead of one memory sector apiece.  Same results either way.  No
                                       counterpart in the reference, whose iterator reads the table by output row
                                       (cumm/conv/sparse_iters.py:280-357). */
  int32_t mask_int_count;           /* tv::gemm::ConvParams::mask_int_count (params.h:413): 32-bit mask words per position.
                                       0 = whatever the descriptor implies: 1, or ceil(kernel_volume / 32) with a
                                       dynamic_mask descriptor - mask_ptr is then [N, words] and mask_out_ptr
                                       [tiles, words], word w holding offsets 32 w .. 32 w + 31, mask_filter applying to
                                       every word (MaskIGemmIteratorMaskLoaderDynamic, cumm/gemm/blockmma/mma.py:78-269).
                                       Any other value than that is an error. */
} CummHipSparseConvArgs;

/* Replaces GemmMainUnitTest.matmul2 below its prelude
 * (cumm/gemm/main.py:1176-1335: dispatch on the descriptor and launch). */
int cumm_hip_gemm(const CummHipGemmDesc *desc, const CummHipGemmArgs *args, void *stream);

/* Replaces ConvMainUnitTest.implicit_gemm2 below its prelude for mask_sparse
 * descriptors (cumm/conv/main.py:483-745). */
int cumm_hip_sparse_conv(const CummHipConvDesc *desc, const CummHipSparseConvArgs *args,
                         void *stream);

/* cumm_hip_sparse_conv for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc) and so cannot provide the
 * workspace that backward-weight needs (split-K semaphores; fp32 partial-sum images and live-tile
 * lists of the split_k_parallel descriptors).  No counterpart in the reference, whose
 * implicit_gemm2 allocates a missing workspace itself (cumm/conv/nvrtc_code.py:183-192).
 * args->workspace / workspace_bytes are ignored: the workspace is an array of
 * CUMM_HIP_STATIC_WORKSPACE_BYTES bytes inside the library, one per GPU, kept until the process
 * ends.  A problem that needs more returns CUMM_HIP_EINVAL.  The call allocates nothing and
 * clears what it needs with kernels (no memset nodes).  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams) race. */
#define CUMM_HIP_STATIC_WORKSPACE_BYTES (8u << 20)
int cumm_hip_sparse_conv_static_ws(const CummHipConvDesc *desc, const CummHipSparseConvArgs *args,
                                   void *stream);

/* GemmAlgoDesp::query_workspace_size / ConvAlgoDesp::query_conv_workspace_size
 * (include/tensorview/gemm/core/params.h:115-132, 286-307): bytes of workspace a launch with these
 * m, n, k (GemmUtils::implicit_gemm_mnk for a convolution, utils.h:62-92) and split_k_slices needs;
 * 0 when it needs none; -1 for a descriptor without a split-K variant and split_k_slices > 1. */
int64_t cumm_hip_query_gemm_workspace(const CummHipGemmDesc *desc, int m, int n, int k, int split_k_slices);
int64_t cumm_hip_query_conv_workspace(const CummHipConvDesc *desc, int m, int n, int k, int split_k_slices,
                                      int kernel_volume);

/* Bytes of workspace with which the fixed-order backward-weight (CummHipSparseConvArgs.deterministic)
 * runs at full width; 256-byte aligned.  With less it uses fewer workgroups, down to a minimum it
 * names in its error.  -1 for arguments it does not take.  (No counterpart in the reference: its
 * fixed-order variant is the serial split-K, sized by query_conv_workspace_size.) */
int64_t cumm_hip_query_wgrad_ordered_workspace(int N, int C, int K, int kernel_volume, int mask_width);

/* GemmMainUnitTest.get_all_algo_desp / ConvMainUnitTest.get_all_conv_algo_desp
 * (cumm/gemm/main.py:914-965, cumm/conv/main.py:467-481): the descriptors this
 * build has kernels for.  Writes at most cap entries, returns the total. */
int cumm_hip_list_gemm_algos(CummHipGemmDesc *out, int cap);
int cumm_hip_list_conv_algos(CummHipConvDesc *out, int cap);

/* 1 if a kernel exists for the descriptor, else 0 (the "found" flag of the
 * dispatch chains, cumm/gemm/main.py:1325-1334, cumm/conv/main.py:734-744). */
int cumm_hip_gemm_supported(const CummHipGemmDesc *desc);
int cumm_hip_conv_supported(const CummHipConvDesc *desc);

/* Text of the last error returned to the calling thread. */
const char *cumm_hip_last_error(void);

/* Which kernels served the calling thread's last successful backward-weight call (a diagnostic for
 * tests, benchmarks and the tuner; no counterpart in the reference, whose descriptor names its one
 * kernel).  LISTS: live-tile lists + balanced units + conversion, three launches on the caller's
 * workspace; SCAN: the (groups, offsets) grid that reads the reduced masks itself + conversion;
 * FIXED_ORDER: the reproducible variant; TILED: the tile GEMM (one slice or serial split-K). */
#define CUMM_HIP_WGRAD_LISTS 2
#define CUMM_HIP_WGRAD_SCAN 3
#define CUMM_HIP_WGRAD_FIXED_ORDER 4
#define CUMM_HIP_WGRAD_TILED 5
int cumm_hip_last_wgrad_path(void);

/* ---- device backend of tv::Tensor / tv::Context (include/tensorview/tensor.h:181-330
 * allocation, :1395 zero_, :1525-1766 copy_/cpu()/cuda(); include/tensorview/contexts/core.h:429-500) */
int cumm_hip_device_count(int *count);                 /* host out-param */
int cumm_hip_malloc(void **ptr, size_t bytes);         /* host out-param */
int cumm_hip_free(void *ptr);
int cumm_hip_host_malloc(void **ptr, size_t bytes);    /* pinned host memory */
int cumm_hip_host_free(void *ptr);
int cumm_hip_memcpy_h2d(void *dst, const void *src_host, size_t bytes, void *stream);
int cumm_hip_memcpy_d2h(void *dst_host, const void *src, size_t bytes, void *stream);
int cumm_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int cumm_hip_memset(void *ptr, int value, size_t bytes, void *stream);
int cumm_hip_stream_create(void **stream);             /* host out-param; default priority */
int cumm_hip_stream_destroy(void *stream);
/* GemmMainUnitTest.stream_synchronize / device_synchronize (cumm/gemm/main.py:1028-1047).
 * Both also report what a kernel could only find out while running: a serial split-K slice whose
 * bounded wait at the semaphore (tv::Semaphore, include/tensorview/gemm/arch/semaphore.h:37-100,
 * waits without a bound) ran out went on without its turn and counted itself; a non-zero count
 * comes back here as CUMM_HIP_ERUNTIME (once; the count is cleared). */
int cumm_hip_stream_synchronize(void *stream);
int cumm_hip_device_synchronize(void);
/* The same count for callers that synchronise by other means (e.g. through torch): reads and
 * clears the current device's count of timed-out split-K slices.  Call after a synchronisation.
 * A mask sort whose look-back gave up since the last report (cumm_hip_sort_by_mask) makes the call
 * return CUMM_HIP_ERUNTIME, with the count of slices still written. */
int cumm_hip_take_async_errors(int32_t *split_k_timeouts);   /* host out-param */
/* Polls a split-K slice makes before it gives up (0 = the default of 2^24, about a second).  For
 * tests of the time-out path and for workloads with very long slices. */
int cumm_hip_set_split_k_spin_limit(int polls);

/* ---- events: tv::CUDAEvent / CUDAKernelTimer (include/tensorview/profile/cuda_profiler.h:97-406) */
int cumm_hip_event_create(void **event);               /* host out-param */
int cumm_hip_event_destroy(void *event);
int cumm_hip_event_record(void *event, void *stream);
int cumm_hip_event_synchronize(void *event);
int cumm_hip_event_elapsed_ms(void *start, void *stop, float *ms); /* host out-param */

/* ---- input preparation for the mask-based kernels (the step before the hot path).
 * The reference does not do this itself: its callers take pair tables and sorted masks from
 * spconv (SpconvOps.generate_subm_conv_inds and sort_1d_by_key, call sites
 * cumm/conv/main_real_spconv.py:91-145); the reference's building block for it is the
 * linear-probing hash table include/tensorview/hash/linear.cu.h:111-840.
 *
 * cumm_hip_subm_pairs: pair tables of a submanifold convolution.
 *   coords [n, 4] int32 (batch, z, y, x), unique; spatial_shape, ksize (odd sizes, kernel volume <= 128),
 *   dilation: 3 ints each (host).  Outputs (device): indices_fwd [kv, n] int32 (-1 = none),
 *   mask_fwd [n] uint32; indices_bwd / mask_fwd / mask_bwd may be NULL.  A kernel volume above 32
 *   has no 32-bit masks (pass NULL for both): its tables feed the per-offset convolution.  Kernel offset k = (kz*KY + ky)*KX + kx,
 *   output o gathers the input at coord[o] + (k_zyx - ksize/2) * dilation.
 *   workspace: at least cumm_hip_subm_pairs_workspace(n) bytes, 16-byte aligned.
 * cumm_hip_sort_by_mask: sorted = stable ascending sort of (mask & mask_filter), argsort = the
 *   permutation; workspace at least cumm_hip_sort_by_mask_workspace(n) bytes.
 *   The sort also counts the light prefix of its result (below) and leaves it in a table inside the
 *   library, on the device, under the address of sorted_mask: a forward / backward-input launch
 *   whose mask_ptr is that array finds it there by itself (no host read, no extra field to fill).
 *   A sort whose bounded waits ran out writes the identity order instead (argsort = 0 .. n-1 with
 *   the masks as they came: valid input for the convolutions, only slower) and the next
 *   synchronising call reports it.
 * cumm_hip_light_prefix: for a sorted mask array (what cumm_hip_sort_by_mask writes, what a
 *   convolution takes as mask_ptr): the number of leading positions, a multiple of 128, in runs of
 *   128 whose two halves of 64 each OR to at most two kernel offsets - a submanifold layer's
 *   centre-only positions lead the ascending order.  Written to *prefix (device memory, one int32;
 *   may be NULL) in stream order - the value is CummHipSparseConvArgs.light_prefix - and into the
 *   library's table like the sort's own count: the call for arrays that another sort made.  The
 *   table is keyed by address, length and filter, holds 256 entries per GPU (a newer array may
 *   replace an older one) and is never needed for correct results.  No counterpart in the reference. */
size_t cumm_hip_subm_pairs_workspace(int n);
int cumm_hip_subm_pairs(const int32_t *coords, int n, const int32_t *spatial_shape, const int32_t *ksize,
                        const int32_t *dilation, int32_t *indices_fwd, int32_t *indices_bwd,
                        uint32_t *mask_fwd, uint32_t *mask_bwd, void *workspace, size_t workspace_bytes,
                        void *stream);
size_t cumm_hip_sort_by_mask_workspace(int n);
int cumm_hip_sort_by_mask(const uint32_t *mask, int n, uint32_t mask_filter, uint32_t *sorted_mask,
                          int32_t *argsort, void *workspace, size_t workspace_bytes, void *stream);
/* The same with a choice of order.  order 0: ascending mask value, what cumm_hip_sort_by_mask and
 * spconv's sort_1d_by_key give.  order 1: ascending number of kernel offsets (set bits of mask &
 * mask_filter), then ascending value; mask_filter must fit 27 bits.  Any order with its masks is valid
 * input of the convolutions (the results are the same rows); this one puts the few positions with many
 * offsets - the rows whose tiles decide how long a launch runs - into a short run at the end, which the
 * forward / backward-input launches then take in half-size tiles (the sort leaves that position in the
 * library's table next to the light prefix), and makes the tiles of the heavy end OR together masks of
 * similar weight (fewer kernel offsets per tile).  No counterpart in the reference. */
int cumm_hip_sort_by_mask_ordered(const uint32_t *mask, int n, uint32_t mask_filter, int order, uint32_t *sorted_mask,
                                  int32_t *argsort, void *workspace, size_t workspace_bytes, void *stream);
int cumm_hip_light_prefix(const uint32_t *sorted_mask, int n, uint32_t mask_filter, int32_t *prefix, void *stream);
/* What the library's table holds for this array, length and filter: *prefix (host) = the light prefix a
 * launch on it would find, *heavy_from (host, may be NULL) = the first position of its heavy end (the first
 * tile of 64 positions whose masks OR to ten or more kernel offsets; n rounded up to 64 = none); -1 each if
 * the table has nothing for the array.  Waits for the stream.  For tests and diagnostics; no launch needs it. */
int cumm_hip_query_light_hint(const uint32_t *sorted_mask, int n, uint32_t mask_filter, int32_t *prefix, int32_t *heavy_from,
                              void *stream);

/* Pair tables of a regular (strided) sparse convolution, in two calls like spconv's
 * generate_conv_inds_mask_stage1 / stage2 (the reference's callers take them from there; its own
 * building block is the same hash table, include/tensorview/hash/linear.cu.h:111-840).  Output
 * shape as ConvProblem.calc_output_dims (cumm/conv/params.py:268-292).  An output site is active
 * iff an input falls into its receptive field; output rows are the active sites in ascending
 * (batch, z, y, x) order; output o gathers the input at o*stride - padding + k_zyx*dilation.
 *
 * cumm_hip_conv_pairs_sites finds the active sites: writes out_shape[3] and *n_out (host) and
 *   SYNCHRONISES the stream once to do so (the caller sizes its tables by n_out).
 * cumm_hip_conv_pairs_fill, with the same coords, geometry and workspace (untouched in between)
 *   and that n_out: out_coords [n_out, 4], indices_fwd [kv, n_out] (both 16-byte aligned), mask_fwd [n_out];
 *   indices_bwd [kv, n_in] / mask_bwd [n_in] may be NULL (indices_bwd[k][i] = the output row that
 *   input i feeds through offset k, -1 = none).
 * batch_size: the batch indices of coords are 0 .. batch_size-1 (others are ignored).  Output
 *   grids of up to 2^33 sites (batch included) are handled with a bitmap of the grid (an eighth
 *   of a byte per site, twice), larger ones with a hash set and a sort: same results.
 * workspace: at least cumm_hip_conv_pairs_workspace(...) bytes (0 = bad geometry), 256-byte aligned.
 * Kernel volumes up to 128; above 32 there are no 32-bit masks: pass NULL for mask_fwd and mask_bwd. */
size_t cumm_hip_conv_pairs_workspace(int n_in, int batch_size, const int32_t *spatial_shape, const int32_t *ksize,
                                     const int32_t *stride, const int32_t *padding, const int32_t *dilation);
int cumm_hip_conv_pairs_sites(const int32_t *coords, int n_in, int batch_size, const int32_t *spatial_shape,
                              const int32_t *ksize, const int32_t *stride, const int32_t *padding,
                              const int32_t *dilation, int32_t *out_shape, int32_t *n_out, void *workspace,
                              size_t workspace_bytes, void *stream);
int cumm_hip_conv_pairs_fill(const int32_t *coords, int n_in, int batch_size, const int32_t *spatial_shape,
                             const int32_t *ksize, const int32_t *stride, const int32_t *padding,
                             const int32_t *dilation, int n_out, int32_t *out_coords, int32_t *indices_fwd,
                             int32_t *indices_bwd, uint32_t *mask_fwd, uint32_t *mask_bwd, void *workspace,
                             size_t workspace_bytes, void *stream);

/* Per-offset pair lists out of a pair table indices [kv, n] (either direction): for every offset k
 * the pairs (indices[k][o], o) with indices[k][o] >= 0, ascending o, packed to the front of
 * pair_in[k, :] / pair_out[k, :] ([kv, n] each), their number in counts[k] (device).  This is the
 * form the per-offset ("native") convolution walks - SparseConvAlgo::kNative,
 * include/tensorview/gemm/core/constants.h:34-38; spconv's indice_pairs [2, kv, N] and
 * indice_num_per_loc, as rebuilt in cumm/conv/main_real_spconv.py:300-326 - and the only one for
 * kernel volumes above 32, which the 32-bit masks cannot describe.
 * workspace: cumm_hip_pair_lists_workspace(kv, n) bytes. */
size_t cumm_hip_pair_lists_workspace(int kv, int n);
int cumm_hip_pair_lists(const int32_t *indices, int kv, int n, int32_t *pair_in, int32_t *pair_out, int32_t *counts,
                        void *workspace, size_t workspace_bytes, void *stream);

/* Masks of a pair table, any kernel volume up to 128: mask [n, words], words = ceil(kv / 32), bit b of
 * word w of output o set wherever indices[32 w + b][o] >= 0 (the layout a dynamic_mask descriptor takes;
 * one word per output for kernel volumes up to 32, where it equals what the table builders write).
 * cumm_hip_sort_by_mask_words: an order for positions with 1 .. 4 mask words - ascending number of offsets,
 * equal masks adjacent (a stable sort by a 32-bit key made of the two) - with sorted_mask [n, words] =
 * the masks in that order and argsort [n]; workspace of cumm_hip_sort_by_mask_words_workspace(n) bytes,
 * 256-byte aligned.  The reference's callers take both steps from spconv for its dynamic-mask kernels
 * (cumm/conv/kernel.py:827-838); any order is valid input, this one keeps the light tiles light. */
int cumm_hip_masks_from_pairs(const int32_t *indices, int kv, int n, uint32_t *mask, void *stream);
size_t cumm_hip_sort_by_mask_words_workspace(int n);
int cumm_hip_sort_by_mask_words(const uint32_t *mask, int n, int words, uint32_t *sorted_mask, int32_t *argsort,
                                void *workspace, size_t workspace_bytes, void *stream);

/* The pair table in the order of the sorted positions: out[k][pos] = indices[k][mask_argsort[pos]] for
 * indices [kv, n] and mask_argsort [n] (an argsort entry outside [0, n) gives -1); out [kv, n], not the
 * table itself.  What CummHipSparseConvArgs.indices_by_position takes: one pass per geometry and sort,
 * after which the entries a tile reads for one kernel offset are consecutive.  No counterpart in the
 * reference (its iterator reads indices[k][mask_argsort[pos]] per access,
 * cumm/conv/sparse_iters.py:280-357). */
int cumm_hip_pairs_by_position(const int32_t *indices, const int32_t *mask_argsort, int kv, int n, int32_t *out,
                               void *stream);

/* ---- stand-alone row gather / scatter-add (the "native" per-offset path around a plain GEMM)
 * cumm_hip_gather_rows: output[i, :] = input[indices[i], :] for i < m; rows of row_bytes bytes
 *   (a multiple of 4), any dtype; an index outside [0, rows_in) gives a row of zeros.
 *   Replaces GatherAll.gather / Gather.gather (cumm/gemm/gather.py:224-256, 482-497).
 * cumm_hip_scatter_add_rows: output[indices[i], :] += input[i, :] for i < m, indices unique; dtype
 *   CUMM_HIP_F32 (the reference's only one), CUMM_HIP_F16 or CUMM_HIP_BF16 (sum formed in fp32,
 *   rounded once); channels * itemsize a multiple of 4; a row whose index is outside
 *   [0, rows_out) is dropped.  Replaces ScatterAll.scatter / Scatter.scatter
 *   (cumm/gemm/gather.py:356-389, 603-617). */
int cumm_hip_gather_rows(void *output, const void *input, const int32_t *indices, int m, int rows_in,
                         size_t row_bytes, void *stream);
int cumm_hip_scatter_add_rows(void *output, const void *input, const int32_t *indices, int m, int rows_out,
                              int channels, int dtype, void *stream);

/* ---- row-wise helpers between launches.  The reference has no counterpart: its callers (spconv's
 * autograd functions and its native convolution) take these steps from torch.
 * cumm_hip_finish_rows: out[r, c] = cvt(act(alpha * acc[r, c] + beta * bias[c])) for an fp32 image
 *   acc [rows, channels] of a result (the per-offset native convolution accumulates in fp32 and
 *   rounds once); out f16 / bf16 (dtype), bias [channels] in that type or NULL, channels % 8 == 0.
 * cumm_hip_relu_backward: dst[i] = out[i] > 0 ? grad[i] : 0 (the gradient through a fused ReLU).
 * cumm_hip_column_sum: dst[c] = cvt(sum over rows of src[r, c]) in fp32, same result from run to
 *   run (the gradient of a bias); workspace of cumm_hip_column_sum_workspace(rows, channels) bytes. */
int cumm_hip_finish_rows(void *out, int dtype, const float *acc, const void *bias, int64_t rows, int channels,
                         float alpha, float beta, int act_type, float act_alpha, void *stream);
int cumm_hip_relu_backward(void *dst, const void *grad, const void *out, size_t elems, int dtype, void *stream);
size_t cumm_hip_column_sum_workspace(int64_t rows, int channels);
int cumm_hip_column_sum(void *dst, const void *src, int64_t rows, int channels, int dtype, void *workspace,
                        size_t workspace_bytes, void *stream);

/* Plain device-to-device copy kernel of `bytes` bytes (16-byte aligned); used to
 * calibrate the HBM traffic counters against a transfer of known size. */
int cumm_hip_copy_kernel(void *dst, const void *src, size_t bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CUMM_HIP_H_ */
