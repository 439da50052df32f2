// C ABI of libcummhip.so: argument checks, kernel selection and launches.
#include "../../include/cumm_hip.h"

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "launch.h"

using namespace cummhip;

namespace {

thread_local std::string g_err;
thread_local int g_wgrad_path = 0;   // CUMM_HIP_WGRAD_* of this thread's last backward-weight call

int fail(int code, const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

int hip_fail(hipError_t e, const char *what) {
  return fail(CUMM_HIP_ERUNTIME, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                   \
  do {                                                  \
    hipError_t e_ = (expr);                             \
    if (e_ != hipSuccess) return hip_fail(e_, #expr);   \
  } while (0)

bool is_float16_like(int dt) { return dt == CUMM_HIP_F16 || dt == CUMM_HIP_BF16; }
int elem_bytes(int dt) { return dt == CUMM_HIP_S8 ? 1 : (is_float16_like(dt) ? 2 : 4); }
int per_vec(int dt) { return 16 / elem_bytes(dt); }
bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// fragments per lane per channel chunk for a contraction of c_in elements
int pick_ks(int c_in, int dt) {
  const int row_bytes = c_in * elem_bytes(dt);
  if (row_bytes <= 64) return 1;
  if (row_bytes <= 128) return 2;
  return 4;
}

// four-byte output of the accumulator type: s8 x s8 -> s32 ("s8,s8,s32,s32,s32",
// cumm/gemm/main.py:350-364,500-523 of the reference), f16 / bf16 -> f32
bool wide_out(const CummHipGemmDesc &d) {
  return d.dtype_a == CUMM_HIP_S8 ? d.dtype_c == CUMM_HIP_S32 : d.dtype_c == CUMM_HIP_F32;
}

// operands of one element type; the output of the same type or of the accumulator's
bool same_dtype3(const CummHipGemmDesc &d) {
  return d.dtype_a == d.dtype_b && (is_float16_like(d.dtype_a) || d.dtype_a == CUMM_HIP_S8) &&
         (d.dtype_a == d.dtype_c || wide_out(d));
}

// accumulator and arithmetic type of the linear combination: f32 / f32; s8 operands accumulate in
// s32 and combine in f32 (s8 output, the requantising epilogues) or in s32 (s32 output)
bool acc_ok(const CummHipGemmDesc &d) {
  if (d.dtype_a == CUMM_HIP_S8)
    return d.dacc == CUMM_HIP_S32 && d.dcomp == (d.dtype_c == CUMM_HIP_S32 ? CUMM_HIP_S32 : CUMM_HIP_F32);
  return d.dacc == CUMM_HIP_F32 && d.dcomp == CUMM_HIP_F32;
}

hipError_t launch_rowgemm(int dt, bool wide, int tm, int tn, int ks, bool wt, const RowGemmParams &p,
                          hipStream_t s) {
  switch (dt) {
  case CUMM_HIP_F16: return wide ? launch_rowgemm_wide_f16(tm, tn, ks, wt, p, s) : launch_rowgemm_f16(tm, tn, ks, wt, p, s);
  case CUMM_HIP_BF16: return wide ? launch_rowgemm_wide_bf16(tm, tn, ks, wt, p, s) : launch_rowgemm_bf16(tm, tn, ks, wt, p, s);
  case CUMM_HIP_S8: return wide ? launch_rowgemm_wide_s8(tm, tn, ks, wt, p, s) : launch_rowgemm_s8(tm, tn, ks, wt, p, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_tilegemm(int dt, bool wide, int tm, int tn, bool xk, bool yk, const TileGemmParams &p,
                           dim3 grid, hipStream_t s) {
  switch (dt) {
  case CUMM_HIP_F16: return wide ? launch_tilegemm_wide_f16(tm, tn, xk, yk, p, grid, s) : launch_tilegemm_f16(tm, tn, xk, yk, p, grid, s);
  case CUMM_HIP_BF16: return wide ? launch_tilegemm_wide_bf16(tm, tn, xk, yk, p, grid, s) : launch_tilegemm_bf16(tm, tn, xk, yk, p, grid, s);
  case CUMM_HIP_S8: return wide ? launch_tilegemm_wide_s8(tm, tn, xk, yk, p, grid, s) : launch_tilegemm_s8(tm, tn, xk, yk, p, grid, s);
  }
  return hipErrorInvalidValue;
}

// bound on the polls of a serial split-K semaphore (cumm_hip_set_split_k_spin_limit)
constexpr int kDefaultSpinLimit = 1 << 24;
std::atomic<int> g_spin_limit{kDefaultSpinLimit};

// byte extent of a row-major 2-D operand for the buffer range checks; false if it does not fit
// below 2 GiB (the kernels use 32-bit offsets and reserve the upper half for "absent")
bool extent32(int64_t rows, int64_t ld, int64_t cols, int esize, uint32_t *out) {
  const int64_t bytes = rows <= 0 ? 0 : ((rows - 1) * ld + cols) * esize;
  if (bytes < 0 || bytes >= (int64_t)1 << 31) return false;
  *out = (uint32_t)bytes;
  return true;
}

// which kernel family serves a GEMM descriptor: 1 rowgemm, 2 tilegemm, 0 none
int gemm_family(const CummHipGemmDesc &d) {
  if (!same_dtype3(d) || !acc_ok(d)) return 0;
  const int tm = d.tile_shape[0], tn = d.tile_shape[1], tk = d.tile_shape[2];
  const int mk = d.dtype_a == CUMM_HIP_S8 ? 64 : 32;
  if (tk != mk) return 0;
  if (d.split_k_parallel) return 0;
  if (d.shuffle_type == CUMM_HIP_SHUFFLE_AC) {
    if (d.trans_a || d.trans_c || d.split_k_serial) return 0;
    return rowgemm_has_tile(tm, tn) ? 1 : 0;
  }
  if (d.shuffle_type == CUMM_HIP_SHUFFLE_AB) {
    if (!d.trans_a || d.trans_b || d.trans_c) return 0;
    return tilegemm_has_tile(tm, tn) ? 2 : 0;
  }
  if (d.shuffle_type == CUMM_HIP_NO_SHUFFLE) return tilegemm_has_tile(tm, tn) ? 2 : 0;
  return 0;
}

int conv_family(const CummHipConvDesc &c) {
  const CummHipGemmDesc &d = c.gemm;
  if (!c.mask_sparse) return 0;
  if (!same_dtype3(d) || !acc_ok(d)) return 0;
  const int tm = d.tile_shape[0], tn = d.tile_shape[1], tk = d.tile_shape[2];
  const int mk = d.dtype_a == CUMM_HIP_S8 ? 64 : 32;
  if (tk != mk) return 0;
  // several mask words per position (kernel volumes above 32): forward and backward-input of
  // two-byte elements on square tiles
  if (c.dynamic_mask && (!(c.op_type == CUMM_HIP_OP_FORWARD || c.op_type == CUMM_HIP_OP_BACKWARD_INPUT) || d.dtype_a == CUMM_HIP_S8 ||
                         wide_out(d) || tm != tn || d.split_k_serial || d.split_k_parallel))
    return 0;
  if (d.split_k_parallel) {
    // only the balanced backward-weight kernel (fp32 atomic partial sums) splits "in parallel"
    if (c.op_type != CUMM_HIP_OP_BACKWARD_WEIGHT || d.dtype_a == CUMM_HIP_S8 || d.split_k_serial || wide_out(d)) return 0;
    if (!d.trans_a || d.trans_b || d.trans_c) return 0;
    return (tm == 64 && tn == 64) ? 3 : 0;
  }
  if (c.is_int8_inference && (d.dtype_a != CUMM_HIP_S8 || c.op_type != CUMM_HIP_OP_FORWARD || wide_out(d))) return 0;
  // (the weight gradient keeps the weight's type, as every kernel of the reference does)
  if (wide_out(d) && c.op_type == CUMM_HIP_OP_BACKWARD_WEIGHT) return 0;
  if (c.op_type == CUMM_HIP_OP_FORWARD || c.op_type == CUMM_HIP_OP_BACKWARD_INPUT) {
    if (d.split_k_serial) return 0;
    return rowgemm_has_tile(tm, tn) ? 1 : 0;
  }
  if (c.op_type == CUMM_HIP_OP_BACKWARD_WEIGHT) {
    if (d.dtype_a == CUMM_HIP_S8) return 0;
    return tilegemm_has_tile(tm, tn) ? 2 : 0;
  }
  return 0;
}

void fill_gemm_desc(CummHipGemmDesc &d, int dt, int ta, int tb, int tc, int tm, int tn, int shuffle,
                    int splitk, bool wide = false, int num_stage = 2) {
  std::memset(&d, 0, sizeof(d));
  d.dtype_a = d.dtype_b = d.dtype_c = dt;
  d.dacc = dt == CUMM_HIP_S8 ? CUMM_HIP_S32 : CUMM_HIP_F32;
  d.dcomp = CUMM_HIP_F32;
  if (wide) {
    d.dtype_c = d.dacc;
    d.dcomp = d.dacc;
  }
  d.trans_a = ta; d.trans_b = tb; d.trans_c = tc;
  const int tk = dt == CUMM_HIP_S8 ? 64 : 32;
  d.tile_shape[0] = tm; d.tile_shape[1] = tn; d.tile_shape[2] = tk;
  d.num_stage = num_stage;
  d.shuffle_type = shuffle;
  d.split_k_serial = splitk;
  d.split_k_parallel = 0;
}

// Zeroes `words` 4-byte words.  Used instead of hipMemsetAsync for semaphores and partial-sum
// images so that a caller may record these entry points into a HIP graph.
__global__ __launch_bounds__(256) void zero_words_kernel(uint32_t *dst, size_t words, int wide) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * 256;
  size_t done = 0;
  if (wide) {   // 16-byte aligned: whole quads first
    const size_t quads = words / 4;
    for (size_t q = i; q < quads; q += stride) reinterpret_cast<v4i *>(dst)[q] = v4i{0, 0, 0, 0};
    done = quads * 4;
  }
  for (size_t w = done + i; w < words; w += stride) dst[w] = 0u;
}

hipError_t zero_device(void *ptr, size_t bytes, hipStream_t s) {
  const size_t words = (bytes + 3) / 4;   // (every size zeroed here is a multiple of 4)
  if (words == 0) return hipSuccess;
  const int wide = aligned16(ptr) ? 1 : 0;
  size_t blocks = ((wide ? words / 4 + 3 : words) + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)blocks), dim3(256), 0, s, reinterpret_cast<uint32_t *>(ptr), words, wide);
  return hipGetLastError();
}

// ---- the library's own scratch memory for cumm_hip_sparse_conv_static_ws: one array per GPU,
// held until the process ends.  In host code the array's name is only a handle for
// hipGetSymbolAddress; kernels and fills take the address that call returns for the current device.
static __device__ __align__(256) unsigned char scratch[CUMM_HIP_STATIC_WORKSPACE_BYTES];
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void **out) {
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(CUMM_HIP_ERUNTIME, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_scratch_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail(CUMM_HIP_ERUNTIME, "hipGetSymbolAddress returned no address for the scratch array");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return CUMM_HIP_OK;
}

// ---- failures that a kernel can only report after the fact.  Word 0 counts the serial split-K
// slices whose bounded semaphore wait ran out (tilegemm.h), word 1 the look-backs of the mask sort
// that ran into their bound (sort_inst.hip).  One array per GPU, like `scratch`: the counts are
// device-wide, whichever stream the launch ran on.  The synchronising entry points take them -
// one kernel that exchanges every word with zero (nothing counted in between is lost) and writes
// what it found into pinned host memory, on a stream of the library's own that does not
// synchronise with the caller's streams - and turn a non-zero count into an error.  Nothing is
// launched or copied while no launch that could report has run since the last look.
static __device__ int32_t async_status[4];
int32_t *g_status_ptr[kMaxDevices] = {};
int32_t *g_status_host[kMaxDevices] = {};       // pinned, four words per GPU
hipStream_t g_status_stream[kMaxDevices] = {};
std::atomic<bool> g_status_armed[kMaxDevices];

__global__ void take_status_kernel(int32_t *status, int32_t *host_words) {
  const int i = threadIdx.x;
  if (i < 4) host_words[i] = atomicExch(&status[i], 0);
}

// The status words of the current device, for a launch that may count into them.
int async_status_ptr(int32_t **out) {
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(CUMM_HIP_ERUNTIME, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_status_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(async_status)));
    if (ptr == nullptr) return fail(CUMM_HIP_ERUNTIME, "hipGetSymbolAddress returned no address for the status words");
    void *host = nullptr;
    HIP_TRY(hipHostMalloc(&host, 4 * sizeof(int32_t), hipHostMallocDefault));
    hipStream_t st = nullptr;
    HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));   // (default priority)
    g_status_host[dev] = reinterpret_cast<int32_t *>(host);
    g_status_stream[dev] = st;
    g_status_ptr[dev] = reinterpret_cast<int32_t *>(ptr);
  }
  g_status_armed[dev].store(true);
  *out = g_status_ptr[dev];
  return CUMM_HIP_OK;
}

// After a synchronisation: anything to report on this device?
int take_async_errors(int32_t *timeouts, int32_t *sort_give_ups = nullptr) {
  *timeouts = 0;
  if (sort_give_ups) *sort_give_ups = 0;
  int dev = -1;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return CUMM_HIP_OK;
  // (disarmed before the look: a launch that arms again after this point is seen by the next look)
  if (!g_status_armed[dev].exchange(false)) return CUMM_HIP_OK;
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  hipLaunchKernelGGL(take_status_kernel, dim3(1), dim3(64), 0, g_status_stream[dev], g_status_ptr[dev], g_status_host[dev]);
  HIP_TRY(hipGetLastError());
  HIP_TRY(hipStreamSynchronize(g_status_stream[dev]));
  *timeouts = g_status_host[dev][0];
  if (sort_give_ups) *sort_give_ups = g_status_host[dev][1];
  return CUMM_HIP_OK;
}

// ---- the table of light-prefix hints (launch.h): one per GPU, like `scratch`
static __device__ __align__(32) int32_t light_hints[kLightHintSlots + 1][8];   // (+ one slot that stays zero)
int32_t *g_hints_ptr[kMaxDevices] = {};

// the slot of a sorted mask array in the current device's table; NULL (and no error) if the
// table cannot be found: hints are optional
int32_t *light_hint_slot_ptr(const void *sorted_mask) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (g_hints_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(light_hints)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_hints_ptr[dev] = reinterpret_cast<int32_t *>(ptr);
  }
  return g_hints_ptr[dev] + 8 * light_hint_slot(sorted_mask);
}

// a slot that names no array: the last one of the table, which light_hint_slot never returns
const int32_t *light_hint_no_slot() {
  const int32_t *first = light_hint_slot_ptr(nullptr);
  return first ? first - 8 * light_hint_slot(nullptr) + 8 * kLightHintSlots : nullptr;
}

int report_async_errors() {
  int32_t timeouts = 0, sort_give_ups = 0;
  if (int rc = take_async_errors(&timeouts, &sort_give_ups)) return rc;
  if (sort_give_ups != 0)
    return fail(CUMM_HIP_ERUNTIME, "mask sort: %d look-back(s) gave up waiting for an earlier chunk; the result of that "
                "sort is invalid", (int)sort_give_ups);
  if (timeouts != 0)
    return fail(CUMM_HIP_ERUNTIME,
                "serial split-K: %d slice(s) gave up waiting for their turn at the semaphore; the results of "
                "those launches are invalid", (int)timeouts);
  return CUMM_HIP_OK;
}

int sparse_conv_impl(const CummHipConvDesc *desc, const CummHipSparseConvArgs *a, void *stream_, void *workspace,
                     size_t workspace_bytes, size_t workspace_cap);

// workspace of the fixed-order backward-weight: live-tile counts (128 bytes), the table of the
// workgroups per (offset, channel block), the live-tile lists, then the slots of partial sums
struct OrderedLayout {
  bool wide;
  int num_red, kblocks, cblocks, combos, keys;
  int64_t max_units;
  size_t block_bytes, lists_at, slots_at;
};
OrderedLayout ordered_layout(int N, int C, int K, int kv, int mask_width) {
  OrderedLayout l;
  l.wide = K > 64 && C > 64;
  const int blk = l.wide ? 128 : 64;
  l.num_red = (N + mask_width - 1) / mask_width;
  l.kblocks = (K + blk - 1) / blk; l.cblocks = (C + blk - 1) / blk;
  l.combos = l.kblocks * l.cblocks; l.keys = kv * l.combos;
  const int qt = kWgradMaxPos / mask_width < 1 ? 1 : kWgradMaxPos / mask_width;
  l.max_units = ((int64_t)((l.num_red + qt - 1) / qt) * kv + kv) * l.combos;
  l.block_bytes = sizeof(float) * blk * blk;
  l.lists_at = 128 + (((size_t)8 * l.keys + 255) & ~(size_t)255);
  l.slots_at = l.lists_at + ((sizeof(int32_t) * (size_t)kv * l.num_red + 255) & ~(size_t)255);
  return l;
}

}  // namespace

extern "C" {

const char *cumm_hip_last_error(void) { return g_err.c_str(); }
int cumm_hip_last_wgrad_path(void) { return g_wgrad_path; }

int cumm_hip_gemm_supported(const CummHipGemmDesc *desc) { return desc && gemm_family(*desc) != 0; }
int cumm_hip_conv_supported(const CummHipConvDesc *desc) { return desc && conv_family(*desc) != 0; }

int64_t cumm_hip_query_gemm_workspace(const CummHipGemmDesc *desc, int m, int n, int k, int split_k_slices) {
  (void)k;
  if (!desc || m < 0 || n < 0 || split_k_slices < 1) return -1;
  if (split_k_slices == 1) return 0;
  const int64_t tiles_m = (m + desc->tile_shape[0] - 1) / desc->tile_shape[0];
  const int64_t tiles_n = (n + desc->tile_shape[1] - 1) / desc->tile_shape[1];
  if (desc->split_k_serial) return (int64_t)sizeof(int32_t) * tiles_m * tiles_n;
  if (desc->split_k_parallel) return (int64_t)4 * m * n * split_k_slices;   // (accumulators are 4 bytes: f32 or s32)
  return -1;
}

int64_t cumm_hip_query_conv_workspace(const CummHipConvDesc *desc, int m, int n, int k, int split_k_slices,
                                      int kernel_volume) {
  if (!desc || kernel_volume < 1) return -1;
  if (!desc->mask_sparse) return cumm_hip_query_gemm_workspace(&desc->gemm, m, n, k, split_k_slices);
  if (m < 0 || n < 0 || split_k_slices < 1) return -1;
  if (split_k_slices == 1) return 0;
  const CummHipGemmDesc &d = desc->gemm;
  const int64_t tiles_m = (m + d.tile_shape[0] - 1) / d.tile_shape[0];
  // backward weight: every kernel offset has its own column blocks (get_spconv_logical_tile_count, utils.h:39-60)
  const int64_t tiles_n = desc->op_type == CUMM_HIP_OP_BACKWARD_WEIGHT
                              ? (int64_t)((n / kernel_volume + d.tile_shape[1] - 1) / d.tile_shape[1]) * kernel_volume
                              : (n + d.tile_shape[1] - 1) / d.tile_shape[1];
  if (d.split_k_serial) return (int64_t)sizeof(int32_t) * tiles_m * tiles_n;
  if (d.split_k_parallel) return (int64_t)4 * m * n * split_k_slices;
  return -1;
}
int64_t cumm_hip_query_wgrad_ordered_workspace(int N, int C, int K, int kernel_volume, int mask_width) {
  if (N < 0 || C <= 0 || K <= 0 || kernel_volume <= 0 || kernel_volume > 32 || mask_width <= 0 || mask_width > kWgradMaxPos)
    return -1;
  const OrderedLayout l = ordered_layout(N, C, K, kernel_volume, mask_width);
  // 512 workgroups: two per compute unit of a 256-unit part (fewer slots only mean fewer workgroups)
  const int64_t wgs = l.max_units < 512 ? l.max_units : 512;
  return (int64_t)l.slots_at + (wgs + l.keys) * (int64_t)l.block_bytes;
}

int cumm_hip_list_gemm_algos(CummHipGemmDesc *out, int cap) {
  std::vector<CummHipGemmDesc> v;
  const int dts[3] = {CUMM_HIP_F16, CUMM_HIP_BF16, CUMM_HIP_S8};
  const int row_tiles[4][2] = {{64, 64}, {128, 64}, {64, 128}, {128, 128}};
  const int sq_tiles[2][2] = {{64, 64}, {128, 128}};
  // every kernel with the output in the operands' type and in the accumulator's (s32 / f32)
  for (int wide = 0; wide < 2; ++wide)
  for (int dt : dts) {
    for (auto &t : row_tiles)
      for (int tb = 0; tb < 2; ++tb) {
        CummHipGemmDesc d;
        fill_gemm_desc(d, dt, 0, tb, 0, t[0], t[1], CUMM_HIP_SHUFFLE_AC, 0, wide != 0);
        d.warp_tile_shape[0] = t[0] / 4; d.warp_tile_shape[1] = t[1]; d.warp_tile_shape[2] = d.tile_shape[2];
        v.push_back(d);
      }
    for (auto &t : sq_tiles) {
      for (int ta = 0; ta < 2; ++ta)
        for (int tb = 0; tb < 2; ++tb)
          for (int tc = 0; tc < 2; ++tc) {
            CummHipGemmDesc d;
            fill_gemm_desc(d, dt, ta, tb, tc, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 1, wide != 0);
            d.warp_tile_shape[0] = t[0] / 2; d.warp_tile_shape[1] = t[1] / 2; d.warp_tile_shape[2] = d.tile_shape[2];
            v.push_back(d);
          }
      CummHipGemmDesc d;
      fill_gemm_desc(d, dt, 1, 0, 0, t[0], t[1], CUMM_HIP_SHUFFLE_AB, 1, wide != 0);
      d.warp_tile_shape[0] = t[0] / 2; d.warp_tile_shape[1] = t[1] / 2; d.warp_tile_shape[2] = d.tile_shape[2];
      v.push_back(d);
    }
  }
  for (int i = 0; i < (int)v.size() && i < cap; ++i) out[i] = v[i];
  return (int)v.size();
}

int cumm_hip_list_conv_algos(CummHipConvDesc *out, int cap) {
  std::vector<CummHipConvDesc> v;
  const int row_tiles[4][2] = {{64, 64}, {128, 64}, {64, 128}, {128, 128}};
  const int sq_tiles[2][2] = {{64, 64}, {128, 128}};
  auto base = [](CummHipConvDesc &c, int op) {
    c.ndim = 3; c.op_type = op; c.mask_sparse = 1; c.increment_k_first = 1; c.dynamic_mask = 0;
    c.is_int8_inference = 0;
  };
  const int fdts[2] = {CUMM_HIP_F16, CUMM_HIP_BF16};
  for (int dt : fdts) {
    for (int wide = 0; wide < 2; ++wide)   // output in the operands' type, then in f32
    for (auto &t : row_tiles)
    // The 128 x 128 tile comes twice: num_stage 3 walks a contraction of more than 128 bytes in
    // 64-byte chunks through three stages of 16 KB (three workgroups per CU: faster where most
    // tiles have few kernel offsets, as in sparse clouds), num_stage 2 in 128-byte chunks through
    // two stages of 32 KB (half as many steps per offset: faster where tiles have many).  Shorter
    // contractions fit one chunk either way.  The three-stage one is listed first.
    for (int stages = (t[0] == 128 && t[1] == 128 ? 3 : 2); stages >= 2; --stages) {
      // forward: A = input [N,C] row major, B = weight [K, kv*C] ("tn"), C = output
      CummHipConvDesc c;
      fill_gemm_desc(c.gemm, dt, 0, 1, 0, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 0, wide != 0, stages);
      c.gemm.warp_tile_shape[0] = t[0] / 4; c.gemm.warp_tile_shape[1] = t[1]; c.gemm.warp_tile_shape[2] = 32;
      base(c, CUMM_HIP_OP_FORWARD);
      v.push_back(c);
      // backward input: A = dOut [N,K], B = weight viewed [kv*K, C] ("tt")
      fill_gemm_desc(c.gemm, dt, 0, 0, 0, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 0, wide != 0, stages);
      c.gemm.warp_tile_shape[0] = t[0] / 4; c.gemm.warp_tile_shape[1] = t[1]; c.gemm.warp_tile_shape[2] = 32;
      base(c, CUMM_HIP_OP_BACKWARD_INPUT);
      v.push_back(c);
    }
    for (auto &t : sq_tiles) {
      // the same two passes with dynamic_mask: ceil(kernel volume / 32) mask words per position
      CummHipConvDesc c;
      fill_gemm_desc(c.gemm, dt, 0, 1, 0, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 0);
      c.gemm.warp_tile_shape[0] = t[0] / 4; c.gemm.warp_tile_shape[1] = t[1]; c.gemm.warp_tile_shape[2] = 32;
      base(c, CUMM_HIP_OP_FORWARD);
      c.dynamic_mask = 1;
      v.push_back(c);
      fill_gemm_desc(c.gemm, dt, 0, 0, 0, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 0);
      c.gemm.warp_tile_shape[0] = t[0] / 4; c.gemm.warp_tile_shape[1] = t[1]; c.gemm.warp_tile_shape[2] = 32;
      base(c, CUMM_HIP_OP_BACKWARD_INPUT);
      c.dynamic_mask = 1;
      v.push_back(c);
    }
    {
      // backward weight, work balanced over live tiles, fp32 atomic partial sums
      CummHipConvDesc c;
      fill_gemm_desc(c.gemm, dt, 1, 0, 0, 64, 64, CUMM_HIP_NO_SHUFFLE, 0);
      c.gemm.split_k_parallel = 1;
      c.gemm.warp_tile_shape[0] = 32; c.gemm.warp_tile_shape[1] = 32; c.gemm.warp_tile_shape[2] = 32;
      base(c, CUMM_HIP_OP_BACKWARD_WEIGHT);
      v.push_back(c);
    }
    for (auto &t : sq_tiles) {
      // backward weight: A = dOut^T [K,N] ("n"), B = input [N, kv*C] ("t"), serial split-K
      CummHipConvDesc c;
      fill_gemm_desc(c.gemm, dt, 1, 0, 0, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 1);
      c.gemm.warp_tile_shape[0] = t[0] / 2; c.gemm.warp_tile_shape[1] = t[1] / 2; c.gemm.warp_tile_shape[2] = 32;
      base(c, CUMM_HIP_OP_BACKWARD_WEIGHT);
      v.push_back(c);
    }
  }
  for (auto &t : row_tiles) {
    // s8 forward: s8 output through alpha / beta, s8 output through the int8-inference epilogue,
    // and the raw s32 accumulators
    for (int kind = 0; kind < 3; ++kind) {
      CummHipConvDesc c;
      fill_gemm_desc(c.gemm, CUMM_HIP_S8, 0, 1, 0, t[0], t[1], CUMM_HIP_NO_SHUFFLE, 0, kind == 2);
      c.gemm.warp_tile_shape[0] = t[0] / 4; c.gemm.warp_tile_shape[1] = t[1]; c.gemm.warp_tile_shape[2] = 64;
      base(c, CUMM_HIP_OP_FORWARD);
      c.is_int8_inference = kind == 1;
      v.push_back(c);
    }
  }
  for (int i = 0; i < (int)v.size() && i < cap; ++i) out[i] = v[i];
  return (int)v.size();
}

// ---------------------------------------------------------------------------------------------
int cumm_hip_gemm(const CummHipGemmDesc *desc, const CummHipGemmArgs *a, void *stream_) {
  if (!desc || !a) return fail(CUMM_HIP_EINVAL, "null descriptor or arguments");
  const CummHipGemmDesc &d = *desc;
  const int fam = gemm_family(d);
  if (fam == 0) return fail(CUMM_HIP_ENOALGO, "can't find any suitable algo for your parameters.");
  hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
  const int dt = d.dtype_a;
  const int pv = per_vec(dt);
  const bool wide = wide_out(d);
  const int pvc = wide ? 4 : pv;             // elements of C / D per 16-byte piece
  const int ebc = wide ? 4 : elem_bytes(dt); // bytes of an element of C / D
  if (wide && d.dtype_c == CUMM_HIP_S32 && a->act_type == CUMM_HIP_ACT_SIGMOID)
    return fail(CUMM_HIP_EINVAL, "no sigmoid in integer arithmetic (s32 output)");
  if (a->m < 0 || a->n < 0 || a->k < 0) return fail(CUMM_HIP_EINVAL, "negative m, n or k");
  if (a->m == 0 || a->n == 0) return CUMM_HIP_OK;
  if (!a->ptr_A || !a->ptr_B || !a->ptr_C) return fail(CUMM_HIP_ERUNTIME, "a,b,c must not empty");
  if (!aligned16(a->ptr_A) || !aligned16(a->ptr_B) || !aligned16(a->ptr_C) ||
      (a->ptr_D && !aligned16(a->ptr_D)))
    return fail(CUMM_HIP_EINVAL, "operand pointers must be 16-byte aligned");
  if (!d.split_k_serial && a->split_k_slices > 1)
    return fail(CUMM_HIP_ERUNTIME, "algo don't support splitk but you provide split_k_slices > 1.");
  if (a->split_k_slices < 1) return fail(CUMM_HIP_EINVAL, "split_k_slices must be >= 1");
  const void *ptr_D = a->ptr_D ? a->ptr_D : a->ptr_C;
  const int64_t ldd = a->ptr_D ? a->stride_D : a->stride_C;

  if (fam == 1) {
    // ShuffleAC: C[c_inds[i]] = act(alpha * A[a_inds[i]] @ op(B) + beta * D[c_inds[i]])
    if (!a->indiceBorC) return fail(CUMM_HIP_ERUNTIME, "a_inds,c_inds tensor must not empty");
    if (a->k % pv || a->n % pv || a->stride_A % pv || a->stride_B % pv || a->stride_C % pvc || ldd % pvc)
      return fail(CUMM_HIP_EINVAL, "this m, n, k isn't supported due to misaligned contiguous dim.");
    RowGemmParams p;
    std::memset(&p, 0, sizeof(p));
    p.A = a->ptr_A; p.W = a->ptr_B; p.C = a->ptr_C; p.D = ptr_D;
    p.out_rows = a->indiceBorC;
    p.gather = a->indiceA;
    p.lda = a->stride_A; p.ldc = a->stride_C; p.ldd = ldd;
    if (d.trans_b) {  // B stored [n, k]
      p.w_stride_n = a->stride_B; p.w_stride_c = 1;
    } else {          // B stored [k, n]
      p.w_stride_n = 1; p.w_stride_c = a->stride_B;
    }
    p.w_stride_k = 0;
    p.n_pos = a->m; p.n_idx = a->m; p.rows_a = a->rows_A; p.rows_c = a->rows_C;
    p.c_in = a->k; p.k_out = a->n; p.kv = 1;
    p.mask_filter = 0xffffffffu;
    p.gather_by_pos = 1;
    p.alpha = a->alpha; p.beta = a->beta; p.act_alpha = a->act_alpha; p.act_beta = a->act_beta;
    p.act = a->act_type;
    p.read_source = a->beta != 0.0f;
    if (p.read_source && ldd != 0 && a->indiceD == nullptr && a->ptr_D != nullptr)
      return fail(CUMM_HIP_EINVAL, "a 2-D D needs the scatter indices (indiceD)");
    const int eb = elem_bytes(dt);
    const int64_t b_rows = d.trans_b ? a->n : a->k, b_cols = d.trans_b ? a->k : a->n;
    if (!extent32(a->rows_A, a->stride_A, a->k, eb, &p.a_bytes) ||
        !extent32(b_rows, a->stride_B, b_cols, eb, &p.w_bytes) ||
        !extent32(a->rows_C, a->stride_C, a->n, ebc, &p.c_bytes) ||
        !extent32(ldd ? a->rows_C : 1, ldd, a->n, ebc, &p.d_bytes))
      return fail(CUMM_HIP_ERUNTIME, "your data exceed int32 range.");
    p.gather_bytes = (uint32_t)a->m * 4u;
    hipError_t e = launch_rowgemm(dt, wide, d.tile_shape[0], d.tile_shape[1], pick_ks(a->k, dt), !d.trans_b, p, stream);
    if (e != hipSuccess) return hip_fail(e, "gather-GEMM-scatter launch");
    return CUMM_HIP_OK;
  }

  // tilegemm: D[m][n] = sum_k Y[m][k] X[n][k]
  TileGemmParams p;
  std::memset(&p, 0, sizeof(p));
  // With trans_c the prelude has already swapped the operands (C^T = B^T A^T,
  // cumm/gemm/nvrtc_code.py:62-67 of the reference): A, B, m, n arrive swapped and only the
  // effective transposes remain to be derived from the descriptor.
  bool ta = d.trans_a, tb = d.trans_b;
  if (d.trans_c) {
    const bool nta = !d.trans_b, ntb = !d.trans_a;
    ta = nta; tb = ntb;
  }
  const void *A = a->ptr_A, *B = a->ptr_B;
  const int64_t lda = a->stride_A, ldb = a->stride_B;
  const int m = a->m, n = a->n;
  if (a->stride_C % 4 || ldd % 4 || n % 4)
    return fail(CUMM_HIP_EINVAL, "this m, n, k isn't supported due to misaligned contiguous dim.");
  if (lda % pv || ldb % pv)
    return fail(CUMM_HIP_EINVAL, "this m, n, k isn't supported due to misaligned contiguous dim.");
  if ((ta ? m : a->k) % pv || (tb ? a->k : n) % pv)
    return fail(CUMM_HIP_EINVAL, "this m, n, k isn't supported due to misaligned contiguous dim.");
  p.Y = A; p.ldy = lda;
  p.X = B; p.ldx = ldb;
  p.C = a->ptr_C; p.D = ptr_D; p.ldc = a->stride_C; p.ldd = ldd;
  p.m = m; p.n = n; p.k = a->k; p.kv = 1; p.mask_filter = 0xffffffffu;
  p.alpha = a->alpha; p.beta = a->beta; p.act_alpha = a->act_alpha; p.act = a->act_type;
  p.split_k = a->split_k_slices;
  p.spin_limit = g_spin_limit.load();
  p.rows_x = 0x7fffffff; p.rows_y = 0x7fffffff;
  bool xk, yk;
  if (d.shuffle_type == CUMM_HIP_SHUFFLE_AB) {
    if (!a->indiceA || !a->indiceBorC) return fail(CUMM_HIP_ERUNTIME, "a_inds,b_inds tensor must not empty");
    yk = false; xk = false;
    p.y_gather = a->indiceA; p.x_gather = a->indiceBorC;
    p.rows_y = a->rows_A; p.rows_x = a->rows_B;
  } else {
    yk = !ta;  // A stored [m, k]
    xk = tb;   // B stored [n, k]
  }
  const int tm = d.tile_shape[0], tn = d.tile_shape[1];
  dim3 grid((m + tm - 1) / tm, (n + tn - 1) / tn, p.split_k);
  if (p.split_k > 1) {
    const size_t need = sizeof(int32_t) * grid.x * grid.y;
    if (!a->workspace || a->workspace_bytes < need)
      return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", need);
    if (reinterpret_cast<uintptr_t>(a->workspace) & 3u) return fail(CUMM_HIP_EINVAL, "workspace must be 4-byte aligned");
    HIP_TRY(zero_device(a->workspace, need, stream));
    p.sem = reinterpret_cast<int32_t *>(a->workspace);
    if (int rc = async_status_ptr(&p.timeouts)) return rc;
  }
  p.split_contig = 1;
  hipError_t e = launch_tilegemm(dt, wide, tm, tn, xk, yk, p, grid, stream);
  if (e != hipSuccess) return hip_fail(e, "GEMM launch");
  return CUMM_HIP_OK;
}

// ---------------------------------------------------------------------------------------------
int cumm_hip_sparse_conv(const CummHipConvDesc *desc, const CummHipSparseConvArgs *a, void *stream_) {
  if (!desc || !a) return fail(CUMM_HIP_EINVAL, "null descriptor or arguments");
  return sparse_conv_impl(desc, a, stream_, a->workspace, a->workspace_bytes, 0);
}

int cumm_hip_sparse_conv_static_ws(const CummHipConvDesc *desc, const CummHipSparseConvArgs *a, void *stream_) {
  if (!desc || !a) return fail(CUMM_HIP_EINVAL, "null descriptor or arguments");
  void *ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  return sparse_conv_impl(desc, a, stream_, ws, CUMM_HIP_STATIC_WORKSPACE_BYTES, CUMM_HIP_STATIC_WORKSPACE_BYTES);
}

}  // extern "C"

namespace {
// workspace_cap != 0: the workspace is the library's own array of that size, and a problem that
// needs more is an argument error (the caller cannot make it larger)
int sparse_conv_impl(const CummHipConvDesc *desc, const CummHipSparseConvArgs *a, void *stream_, void *workspace,
                     size_t workspace_bytes, size_t workspace_cap) {
  const CummHipConvDesc &c = *desc;
  const CummHipGemmDesc &d = c.gemm;
  const int fam = conv_family(c);
  if (fam == 0) return fail(CUMM_HIP_ENOALGO, "can't find any suitable algo for your parameters.");
  hipStream_t stream = reinterpret_cast<hipStream_t>(stream_);
  const int dt = d.dtype_a;
  const int pv = per_vec(dt);
  const bool wide = wide_out(d);
  if (wide && d.dtype_c == CUMM_HIP_S32 && a->act_type == CUMM_HIP_ACT_SIGMOID)
    return fail(CUMM_HIP_EINVAL, "no sigmoid in integer arithmetic (s32 output)");
  const int kv = a->kernel_volume;
  if (a->N < 0 || a->C <= 0 || a->K <= 0 || kv <= 0) return fail(CUMM_HIP_EINVAL, "bad N, C, K or kernel volume");
  if (a->mode != CUMM_HIP_CONV_CROSS_CORRELATION)
    return fail(CUMM_HIP_EINVAL, "mode must be cross-correlation (1): the mask-based kernels implement nothing else");
  if (a->groups != 1) return fail(CUMM_HIP_EINVAL, "grouped convolution has no kernel (groups must be 1)");
  // mask words per position: one, or with a dynamic_mask descriptor ceil(kv / 32) as in the
  // reference's kernels (cumm/conv/kernel.py:827-838)
  const int mask_words = c.dynamic_mask ? (kv + 31) / 32 : 1;
  if (kv > 32 && !c.dynamic_mask) return fail(CUMM_HIP_EINVAL, "kernel volume > 32 needs a dynamic_mask descriptor");
  if (kv > kMaxKernelVolume) return fail(CUMM_HIP_EINVAL, "kernel volume above %d", kMaxKernelVolume);
  if (a->mask_int_count != 0 && a->mask_int_count != mask_words)
    return fail(CUMM_HIP_EINVAL, "mask_int_count must be %d for this descriptor and kernel volume", mask_words);
  if (!a->ptr_A || !a->ptr_B || !a->ptr_C) return fail(CUMM_HIP_ERUNTIME, "input, weight and output must not be empty");
  if (!a->indice_ptr || !a->mask_ptr || !a->mask_argsort_ptr)
    return fail(CUMM_HIP_ERUNTIME, "indices, mask and mask_argsort must not be empty");
  if (!aligned16(a->ptr_A) || !aligned16(a->ptr_B) || !aligned16(a->ptr_C) || (a->ptr_D && !aligned16(a->ptr_D)))
    return fail(CUMM_HIP_EINVAL, "operand pointers must be 16-byte aligned");
  if (a->C % pv || a->K % pv) return fail(CUMM_HIP_ERUNTIME, "C and K must be multiples of %d for this element type", pv);
  if (!d.split_k_serial && !d.split_k_parallel && a->split_k_slices > 1)
    return fail(CUMM_HIP_ERUNTIME, "algo don't support splitk but you provide split_k_slices > 1.");
  if (a->N == 0) return CUMM_HIP_OK;
  const void *ptr_D = a->ptr_D ? a->ptr_D : a->ptr_C;

  if (fam == 1) {
    const bool fwd = c.op_type == CUMM_HIP_OP_FORWARD;
    RowGemmParams p;
    std::memset(&p, 0, sizeof(p));
    p.A = a->ptr_A; p.W = a->ptr_B; p.C = a->ptr_C; p.D = ptr_D;
    p.out_rows = a->mask_argsort_ptr;
    p.gather = a->indice_ptr;
    p.mask = a->mask_ptr;
    p.mask_out = fwd ? a->mask_out_ptr : nullptr;
    p.n_pos = a->N; p.n_idx = a->N; p.kv = kv;
    p.mask_filter = a->mask_filter;
    if (fwd) {
      // input [rows_in, C] x weight [K, kv, C] -> output [rows_out, K]
      p.lda = a->C; p.ldc = a->K; p.c_in = a->C; p.k_out = a->K;
      p.rows_a = a->rows_in; p.rows_c = a->rows_out;
      p.w_stride_n = (int64_t)kv * a->C; p.w_stride_k = a->C; p.w_stride_c = 1;
    } else {
      // dOut [rows_out, K] x weight -> dIn [rows_in, C]; contraction over K
      p.lda = a->K; p.ldc = a->C; p.c_in = a->K; p.k_out = a->C;
      p.rows_a = a->rows_out; p.rows_c = a->rows_in;
      p.w_stride_n = 1; p.w_stride_k = a->C; p.w_stride_c = (int64_t)kv * a->C;
      p.reverse_mask = a->reverse_mask;
      p.exit_on_empty = 1;
    }
    p.ldd = a->d_is_bias ? 0 : p.ldc;
    p.alpha = a->alpha; p.beta = a->beta; p.act_alpha = a->act_alpha; p.act_beta = a->act_beta;
    p.act = a->act_type;
    p.read_source = a->beta != 0.0f;
    // (the hint only moves work between tile shapes; whatever it says the kernel covers every position once)
    p.pair_tiles = a->light_prefix > 0 && !a->ungated_rows ? a->light_prefix / 128 : 0;
    // without a count from the caller: what input preparation left in the table for this mask array;
    // with one, or without a table, a slot that names no array (the kernel reads it in any case)
    if (a->light_prefix >= 0 && !a->ungated_rows && mask_words == 1 && d.tile_shape[0] == 64 && d.tile_shape[1] == 64)
      p.hint_slot = a->light_prefix == 0 ? light_hint_slot_ptr(a->mask_ptr) : light_hint_no_slot();
    p.ungated_rows = a->ungated_rows != 0;
    p.mask_words = mask_words;
    if (mask_words > 1) {
      p.pair_tiles = 0;
      if ((int64_t)a->N * mask_words * 4 >= (int64_t)1 << 31) return fail(CUMM_HIP_ERUNTIME, "your data exceed int32 range.");
    }
    p.gather_by_pos = a->indices_by_position != 0;
    p.n_mask_out = p.mask_out ? (a->N + d.tile_shape[0] - 1) / d.tile_shape[0] * mask_words : 0;
    if (c.is_int8_inference) {
      if (!a->bias_pointer || !a->scale_pointer)
        return fail(CUMM_HIP_ERUNTIME, "int8 inference must have both scale and bias");
      p.int8_epilogue = 1;
      p.scale = reinterpret_cast<const float *>(a->scale_pointer);
      p.bias = reinterpret_cast<const float *>(a->bias_pointer);
      p.ldd = p.ldc;  // the only source of the int8 epilogue is output_add (or the output itself)
    }
    const int eb = elem_bytes(dt), ebc = wide ? 4 : eb;
    if (!extent32(p.rows_a, p.lda, p.c_in, eb, &p.a_bytes) ||
        !extent32((int64_t)a->K * kv, a->C, a->C, eb, &p.w_bytes) ||
        !extent32(p.rows_c, p.ldc, p.k_out, ebc, &p.c_bytes) ||
        !extent32(p.ldd ? p.rows_c : 1, p.ldd, p.k_out, ebc, &p.d_bytes) ||
        (int64_t)kv * a->N * 4 >= (int64_t)1 << 31)
      return fail(CUMM_HIP_ERUNTIME, "your data exceed int32 range.");
    p.gather_bytes = (uint32_t)((int64_t)kv * a->N * 4);
    p.stream_stores = p.c_bytes <= kStreamStoreMaxBytes;
    p.small_stages = d.num_stage >= 3;
    hipError_t e = launch_rowgemm(dt, wide, d.tile_shape[0], d.tile_shape[1], pick_ks(p.c_in, dt), !fwd, p, stream);
    if (e != hipSuccess) return hip_fail(e, "sparse conv launch");
    return CUMM_HIP_OK;
  }

  // backward weight: dW[K, kv, C]; A = dOut [N, K], B = input [*, C]
  const int tm = d.tile_shape[0], tn = d.tile_shape[1], tk = d.tile_shape[2];
  if (a->mask_width <= 0 || a->mask_width % tk) return fail(CUMM_HIP_ERUNTIME, "mask_width must be a positive multiple of tile k");
  if (fam == 3 && a->deterministic && !(a->split_k_slices > 1 && a->mask_width <= kWgradMaxPos))
    return fail(CUMM_HIP_EINVAL, "the fixed-order backward-weight needs split_k_slices > 1 and mask_width <= %d", kWgradMaxPos);
  // The fixed-order variant (partial sums in slots, added up in a fixed order, see
  // WgradParams::key_range) runs when the caller asks for it, and by itself where it is also the
  // faster one: with many more units than resident workgroups a workgroup carries its sum through
  // its run of units in registers instead of adding every unit's block into the image with atomics
  // (0.25 against 0.29 ms for C = K = 128 at 1 M voxels) - if the workspace has room for all of its
  // workgroups.
  bool ordered = fam == 3 && a->deterministic;
  if (fam == 3 && a->split_k_slices > 1 && a->mask_width <= kWgradMaxPos) {
    const OrderedLayout lay = ordered_layout(a->N, a->C, a->K, kv, a->mask_width);
    const int qt = kWgradMaxPos / a->mask_width < 1 ? 1 : kWgradMaxPos / a->mask_width;
    const bool fits32 = (int64_t)a->rows_out * a->K * 2 < (int64_t)1 << 31 && (int64_t)a->rows_in * a->C * 2 < (int64_t)1 << 31 &&
                        (int64_t)kv * a->N * 4 < (int64_t)1 << 31;
    const int64_t unit_bound = ((int64_t)(lay.num_red + qt - 1) / qt + 1) * kv * (((int64_t)a->K + 63) / 64) * (((int64_t)a->C + 63) / 64);
    const bool size_ok = fits32 && unit_bound < ((int64_t)1 << 22) && lay.num_red < (1 << 22);
    const bool aligned = (reinterpret_cast<uintptr_t>(workspace) & 255u) == 0;
    if (ordered && !size_ok)
      return fail(CUMM_HIP_EINVAL, "the fixed-order backward-weight does not take a problem of this size; use a split_k_serial descriptor");
    if (ordered && !aligned) return fail(CUMM_HIP_EINVAL, "workspace must be 256-byte aligned");
    int64_t wgs = 0;
    if (size_ok && aligned) {
      const int resident = dt == CUMM_HIP_F16 ? wgrad_ordered_resident_f16(lay.wide) : wgrad_ordered_resident_bf16(lay.wide);
      if (resident < 1) return hip_fail(hipGetLastError(), "occupancy query");
      const int64_t full = resident < lay.max_units ? resident : lay.max_units;
      wgs = full;
      const int64_t have = workspace && workspace_bytes > lay.slots_at ? (int64_t)((workspace_bytes - lay.slots_at) / lay.block_bytes) : 0;
      if (have - lay.keys + 1 < wgs) wgs = have - lay.keys + 1;
      const int64_t by_descriptor = (((int64_t)1 << 32) - 1) / (int64_t)lay.block_bytes - lay.keys + 1;
      if (by_descriptor < wgs) wgs = by_descriptor;
      if (!ordered && wgs == full && (lay.num_red + qt - 1) / qt >= resident) ordered = true;
    }
    const size_t least = lay.slots_at + (size_t)lay.keys * lay.block_bytes;
    if (ordered && workspace_cap && least > workspace_cap)
      return fail(CUMM_HIP_EINVAL, "this problem needs %zu bytes of workspace, the static one holds %zu", least, workspace_cap);
    if (ordered && wgs < 1) return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", least);
    if (ordered) {
    char *base = reinterpret_cast<char *>(workspace);
    WgradParams w;
    std::memset(&w, 0, sizeof(w));
    w.dout = a->ptr_A; w.inp = a->ptr_B; w.scratch = reinterpret_cast<float *>(base + lay.slots_at);
    w.argsort = a->mask_argsort_ptr; w.indices = a->indice_ptr; w.red_mask = a->mask_ptr;
    w.num_red = lay.num_red; w.mask_width = a->mask_width; w.mask_filter = a->mask_filter;
    w.n_pos = a->N; w.n_idx = a->N; w.rows_x = a->rows_in; w.rows_y = a->rows_out;
    w.K = a->K; w.C = a->C; w.kv = kv; w.tiles_per_wg = qt;
    w.images = 1;
    w.live_cnt = reinterpret_cast<int32_t *>(base);
    w.key_range = reinterpret_cast<int32_t *>(base + 128);
    w.live_list = reinterpret_cast<int32_t *>(base + lay.lists_at);
    WgradPrepareParams pre;
    std::memset(&pre, 0, sizeof(pre));
    pre.red_mask = w.red_mask; pre.num_red = w.num_red; pre.kv = kv; pre.mask_filter = w.mask_filter;
    pre.live_cnt = reinterpret_cast<int32_t *>(base);
    pre.live_list = reinterpret_cast<int32_t *>(base + lay.lists_at);
    WgradOrderedParams f;
    std::memset(&f, 0, sizeof(f));
    f.slots = w.scratch; f.key_range = w.key_range; f.dw = a->ptr_C; f.src = ptr_D;
    f.total = (int64_t)a->K * kv * a->C; f.K = a->K; f.C = a->C; f.kv = kv;
    f.block_k = f.block_c = lay.wide ? 128 : 64;
    f.cblocks = lay.cblocks; f.per_r = lay.combos;
    f.mask_filter = a->mask_filter; f.alpha = a->alpha; f.beta = a->beta;
    f.slots_bytes = (uint32_t)((wgs + lay.keys - 1) * (int64_t)lay.block_bytes);
    hipError_t e = dt == CUMM_HIP_F16 ? launch_wgrad_ordered_f16(w, pre, f, lay.wide, (int)wgs, stream)
                                      : launch_wgrad_ordered_bf16(w, pre, f, lay.wide, (int)wgs, stream);
    if (e == hipErrorNotSupported)
      return fail(CUMM_HIP_ERUNTIME, "the fixed-order backward-weight kernel of this build uses scratch memory, which its "
                  "hand-counted waits do not allow; use a split_k_serial descriptor");
    if (e != hipSuccess) return hip_fail(e, "sparse conv wgrad launch");
    g_wgrad_path = CUMM_HIP_WGRAD_FIXED_ORDER;
    return CUMM_HIP_OK;
    }
  }
  if (fam == 3 && a->split_k_slices > 1 && a->mask_width <= kWgradMaxPos) {
    const size_t need = sizeof(float) * (size_t)a->K * kv * a->C;
    if (workspace_cap && need > workspace_cap)
      return fail(CUMM_HIP_EINVAL, "this problem needs %zu bytes of workspace, the static one holds %zu", need, workspace_cap);
    if (!workspace || workspace_bytes < need)
      return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", need);
    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return fail(CUMM_HIP_EINVAL, "workspace must be 16-byte aligned");
    WgradParams w;
    std::memset(&w, 0, sizeof(w));
    w.dout = a->ptr_A; w.inp = a->ptr_B; w.scratch = reinterpret_cast<float *>(workspace);
    w.argsort = a->mask_argsort_ptr; w.indices = a->indice_ptr; w.red_mask = a->mask_ptr;
    w.num_red = (a->N + a->mask_width - 1) / a->mask_width; w.mask_width = a->mask_width;
    w.mask_filter = a->mask_filter;
    w.n_pos = a->N; w.n_idx = a->N; w.rows_x = a->rows_in; w.rows_y = a->rows_out;
    w.K = a->K; w.C = a->C; w.kv = kv;
    int qt = kWgradMaxPos / a->mask_width;
    if (qt < 1) qt = 1;
    w.tiles_per_wg = qt;
    WgradFinalizeParams f;
    std::memset(&f, 0, sizeof(f));
    f.scratch = w.scratch; f.dw = a->ptr_C; f.src = ptr_D;
    f.total = (int64_t)a->K * kv * a->C; f.C = a->C; f.kv = kv; f.mask_filter = a->mask_filter;
    f.alpha = a->alpha; f.beta = a->beta;
    // With room behind the fp32 image for the per-offset live-tile lists, a prepare kernel makes
    // them (and zeroes the image) and the unit-walking kernel runs; as many more copies of the
    // image as fit (at most 8, at most split_k_slices) spread its atomics.  Otherwise the image is
    // zeroed here and every workgroup of the scanning kernel reads the mask itself.
    const size_t image_bytes = (need + 255) & ~(size_t)255;
    const size_t lists_bytes = 128 + sizeof(int32_t) * (size_t)kv * w.num_red;
    int images = 0;
    for (int s = 8; s >= 1 && !images; s >>= 1)
      if (s <= a->split_k_slices && workspace_bytes >= s * image_bytes + lists_bytes &&
          (uint64_t)s * image_bytes < ((uint64_t)1 << 32))   // (the finalize kernel reads them through one descriptor)
        images = s;
    const bool fits32 = (int64_t)a->rows_out * a->K * 2 < (int64_t)1 << 31 && (int64_t)a->rows_in * a->C * 2 < (int64_t)1 << 31 &&
                        (int64_t)kv * a->N * 4 < (int64_t)1 << 31;
    WgradPrepareParams pre;
    std::memset(&pre, 0, sizeof(pre));
    w.images = f.images = 1;
    w.image_floats = f.image_floats = (int64_t)(image_bytes / sizeof(float));
    // (the unit-walking kernel divides unit numbers with a float reciprocal: exact below 2^22)
    const int64_t unit_bound = ((int64_t)(w.num_red + qt - 1) / qt + 1) * kv * (((int64_t)a->K + 63) / 64) * (((int64_t)a->C + 63) / 64);
    if (images && fits32 && unit_bound < ((int64_t)1 << 22) && w.num_red < (1 << 22)) {
      char *base = reinterpret_cast<char *>(workspace);
      const size_t lists_at = images * image_bytes;
      pre.scratch = w.scratch; pre.scratch_floats = (int64_t)(lists_at / sizeof(float));
      pre.red_mask = w.red_mask; pre.num_red = w.num_red; pre.kv = kv; pre.mask_filter = w.mask_filter;
      pre.live_cnt = reinterpret_cast<int32_t *>(base + lists_at);
      pre.live_list = reinterpret_cast<int32_t *>(base + lists_at + 128);
      w.live_cnt = pre.live_cnt; w.live_list = pre.live_list;
      w.images = f.images = images;
      w.image_floats = f.image_floats = (int64_t)(image_bytes / sizeof(float));
    } else {
      HIP_TRY(zero_device(workspace, need, stream));
    }
    hipError_t e = dt == CUMM_HIP_F16 ? launch_wgrad_atomic_f16(w, pre, f, stream) : launch_wgrad_atomic_bf16(w, pre, f, stream);
    if (e == hipErrorNotSupported && w.live_list != nullptr) {
      // the unit-walking kernel failed its load-time check (see counted_waits_hold): the scanning
      // kernel on one image, zeroed here
      w.live_cnt = nullptr; w.live_list = nullptr;
      w.images = f.images = 1;
      HIP_TRY(zero_device(workspace, need, stream));
      e = dt == CUMM_HIP_F16 ? launch_wgrad_atomic_f16(w, pre, f, stream) : launch_wgrad_atomic_bf16(w, pre, f, stream);
    }
    if (e != hipSuccess) return hip_fail(e, "sparse conv wgrad launch");
    g_wgrad_path = w.live_list != nullptr ? CUMM_HIP_WGRAD_LISTS : CUMM_HIP_WGRAD_SCAN;
    return CUMM_HIP_OK;
  }
  TileGemmParams p;
  std::memset(&p, 0, sizeof(p));
  p.Y = a->ptr_A; p.ldy = a->K;       // dOut rows, m = K
  p.X = a->ptr_B; p.ldx = a->C;       // input rows, n = C
  p.C = a->ptr_C; p.D = ptr_D;
  p.ldc = (int64_t)kv * a->C; p.ldd = p.ldc; p.c_off = a->C;
  p.y_gather = a->mask_argsort_ptr;
  p.x_gather = a->indice_ptr; p.x_gather_via_y = 1;
  p.red_mask = a->mask_ptr;
  p.num_red_mask = (a->N + a->mask_width - 1) / a->mask_width;
  p.mask_width = a->mask_width;
  p.mask_filter = a->mask_filter;
  p.m = a->K; p.n = a->C; p.k = a->N; p.n_idx = a->N;
  p.rows_y = a->rows_out; p.rows_x = a->rows_in;
  p.kv = kv;
  p.alpha = a->alpha; p.beta = a->beta; p.act_alpha = a->act_alpha; p.act = a->act_type;
  p.split_k = a->split_k_slices < 1 ? 1 : a->split_k_slices;
  if (fam == 3) p.split_k = 1;   // a single slice needs no partial sums: plain tiled kernel
  p.spin_limit = g_spin_limit.load();
  const int n_tiles = (a->C + tn - 1) / tn;
  dim3 grid((a->K + tm - 1) / tm, n_tiles * kv, p.split_k);
  if (p.split_k > 1) {
    const size_t need = sizeof(int32_t) * grid.x * grid.y;
    if (workspace_cap && need > workspace_cap)
      return fail(CUMM_HIP_EINVAL, "this problem needs %zu bytes of workspace, the static one holds %zu", need, workspace_cap);
    if (!workspace || workspace_bytes < need)
      return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", need);
    if (reinterpret_cast<uintptr_t>(workspace) & 3u) return fail(CUMM_HIP_EINVAL, "workspace must be 4-byte aligned");
    HIP_TRY(zero_device(workspace, need, stream));
    p.sem = reinterpret_cast<int32_t *>(workspace);
    if (int rc = async_status_ptr(&p.timeouts)) return rc;
  }
  hipError_t e = launch_tilegemm(dt, false, tm, tn, false, false, p, grid, stream);
  if (e != hipSuccess) return hip_fail(e, "sparse conv wgrad launch");
  g_wgrad_path = CUMM_HIP_WGRAD_TILED;
  return CUMM_HIP_OK;
}
}  // namespace

extern "C" {

// ---------------------------------------------------------------------------------------------
int cumm_hip_device_count(int *count) {
  if (!count) return fail(CUMM_HIP_EINVAL, "null out-param");
  hipError_t e = hipGetDeviceCount(count);
  if (e != hipSuccess) { *count = 0; return hip_fail(e, "hipGetDeviceCount"); }
  return CUMM_HIP_OK;
}
int cumm_hip_malloc(void **ptr, size_t bytes) {
  if (!ptr) return fail(CUMM_HIP_EINVAL, "null out-param");
  *ptr = nullptr;
  if (bytes == 0) return CUMM_HIP_OK;
  HIP_TRY(hipMalloc(ptr, bytes));
  return CUMM_HIP_OK;
}
int cumm_hip_free(void *ptr) {
  if (ptr) HIP_TRY(hipFree(ptr));
  return CUMM_HIP_OK;
}
int cumm_hip_host_malloc(void **ptr, size_t bytes) {
  if (!ptr) return fail(CUMM_HIP_EINVAL, "null out-param");
  *ptr = nullptr;
  if (bytes == 0) return CUMM_HIP_OK;
  HIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
  return CUMM_HIP_OK;
}
int cumm_hip_host_free(void *ptr) {
  if (ptr) HIP_TRY(hipHostFree(ptr));
  return CUMM_HIP_OK;
}
int cumm_hip_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return CUMM_HIP_OK;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, reinterpret_cast<hipStream_t>(stream)));
  HIP_TRY(hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)));
  return CUMM_HIP_OK;
}
int cumm_hip_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return CUMM_HIP_OK;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, reinterpret_cast<hipStream_t>(stream)));
  HIP_TRY(hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)));
  return CUMM_HIP_OK;
}
int cumm_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return CUMM_HIP_OK;
  HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, reinterpret_cast<hipStream_t>(stream)));
  return CUMM_HIP_OK;
}
int cumm_hip_memset(void *ptr, int value, size_t bytes, void *stream) {
  if (bytes == 0) return CUMM_HIP_OK;
  HIP_TRY(hipMemsetAsync(ptr, value, bytes, reinterpret_cast<hipStream_t>(stream)));
  return CUMM_HIP_OK;
}
int cumm_hip_stream_create(void **stream) {
  if (!stream) return fail(CUMM_HIP_EINVAL, "null out-param");
  hipStream_t s;
  HIP_TRY(hipStreamCreate(&s));
  *stream = s;
  return CUMM_HIP_OK;
}
int cumm_hip_stream_destroy(void *stream) {
  HIP_TRY(hipStreamDestroy(reinterpret_cast<hipStream_t>(stream)));
  return CUMM_HIP_OK;
}
int cumm_hip_stream_synchronize(void *stream) {
  HIP_TRY(hipStreamSynchronize(reinterpret_cast<hipStream_t>(stream)));
  return report_async_errors();
}
int cumm_hip_device_synchronize(void) {
  HIP_TRY(hipDeviceSynchronize());
  return report_async_errors();
}
int cumm_hip_take_async_errors(int32_t *split_k_timeouts) {
  if (!split_k_timeouts) return fail(CUMM_HIP_EINVAL, "null out-param");
  int32_t sort_give_ups = 0;
  if (int rc = take_async_errors(split_k_timeouts, &sort_give_ups)) return rc;
  if (sort_give_ups != 0)
    return fail(CUMM_HIP_ERUNTIME, "mask sort: %d look-back(s) gave up waiting for an earlier chunk; the result of that "
                "sort is invalid", (int)sort_give_ups);
  return CUMM_HIP_OK;
}
int cumm_hip_set_split_k_spin_limit(int polls) {
  if (polls < 0) return fail(CUMM_HIP_EINVAL, "the number of polls must not be negative (0 = the default)");
  g_spin_limit.store(polls == 0 ? kDefaultSpinLimit : polls);
  return CUMM_HIP_OK;
}
int cumm_hip_event_create(void **event) {
  if (!event) return fail(CUMM_HIP_EINVAL, "null out-param");
  hipEvent_t e;
  HIP_TRY(hipEventCreate(&e));
  *event = e;
  return CUMM_HIP_OK;
}
int cumm_hip_event_destroy(void *event) {
  HIP_TRY(hipEventDestroy(reinterpret_cast<hipEvent_t>(event)));
  return CUMM_HIP_OK;
}
int cumm_hip_event_record(void *event, void *stream) {
  HIP_TRY(hipEventRecord(reinterpret_cast<hipEvent_t>(event), reinterpret_cast<hipStream_t>(stream)));
  return CUMM_HIP_OK;
}
int cumm_hip_event_synchronize(void *event) {
  HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(event)));
  return CUMM_HIP_OK;
}
int cumm_hip_event_elapsed_ms(void *start, void *stop, float *ms) {
  if (!ms) return fail(CUMM_HIP_EINVAL, "null out-param");
  HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(start), reinterpret_cast<hipEvent_t>(stop)));
  return CUMM_HIP_OK;
}

__global__ void copy16_kernel(v4i *dst, const v4i *src, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) dst[i] = src[i];
}

static uint32_t pairs_slots(int n) {
  uint32_t slots = 1024;
  while (slots < 2u * (uint32_t)(n > 0 ? n : 0)) slots <<= 1;   // load factor at most one half
  return slots;
}

// hash table slots (16 bytes each), then one presence word per slot pair
size_t cumm_hip_subm_pairs_workspace(int n) { return (size_t)pairs_slots(n) * 16 + (size_t)pairs_slots(n) * 4; }

int cumm_hip_subm_pairs(const int32_t *coords, int n, const int32_t *spatial_shape, const int32_t *ksize,
                        const int32_t *dilation, int32_t *indices_fwd, int32_t *indices_bwd,
                        uint32_t *mask_fwd, uint32_t *mask_bwd, void *workspace, size_t workspace_bytes,
                        void *stream) {
  if (n < 0 || !spatial_shape || !ksize || !dilation) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (n == 0) return CUMM_HIP_OK;
  if (n > (1 << 30)) return fail(CUMM_HIP_EINVAL, "too many voxels");
  if (!coords || !indices_fwd) return fail(CUMM_HIP_EINVAL, "coords and indices_fwd must not be empty");
  if (!aligned16(coords) || !aligned16(workspace)) return fail(CUMM_HIP_EINVAL, "coords and workspace must be 16-byte aligned");
  const int64_t kv = (int64_t)ksize[0] * ksize[1] * ksize[2];
  if (ksize[0] < 1 || ksize[1] < 1 || ksize[2] < 1 || kv > kMaxKernelVolume)
    return fail(CUMM_HIP_EINVAL, "kernel volume must be 1..%d", kMaxKernelVolume);
  if (kv > 32 && (mask_fwd || mask_bwd))
    return fail(CUMM_HIP_EINVAL, "kernel volumes above 32 have no 32-bit masks: pass NULL for mask_fwd and mask_bwd");
  // indices_bwd[k] = indices_fwd[kv-1-k] and the bit-reversed masks hold only when offset kv-1-k is
  // the negative of offset k, i.e. for odd kernel sizes
  if (!(ksize[0] & 1) || !(ksize[1] & 1) || !(ksize[2] & 1))
    return fail(CUMM_HIP_EINVAL, "submanifold convolution needs odd kernel sizes");
  for (int d = 0; d < 3; ++d)
    if (spatial_shape[d] < 1 || dilation[d] < 1) return fail(CUMM_HIP_EINVAL, "spatial_shape and dilation must be positive");
  if (!workspace || workspace_bytes < cumm_hip_subm_pairs_workspace(n))
    return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", cumm_hip_subm_pairs_workspace(n));
  SubmPairsParams p;
  std::memset(&p, 0, sizeof(p));
  p.coords = coords; p.n = n; p.kv = (int)kv;
  for (int d = 0; d < 3; ++d) p.shape[d] = spatial_shape[d];
  for (int k = 0; k < (int)kv; ++k) {
    const int kz = k / (ksize[1] * ksize[2]), ky = (k / ksize[2]) % ksize[1], kx = k % ksize[2];
    p.off[k][0] = (kz - ksize[0] / 2) * dilation[0];
    p.off[k][1] = (ky - ksize[1] / 2) * dilation[1];
    p.off[k][2] = (kx - ksize[2] / 2) * dilation[2];
  }
  p.ind_f = indices_fwd; p.ind_b = indices_bwd; p.mask_f = mask_fwd; p.mask_b = mask_bwd;
  p.table = workspace; p.slot_mask = pairs_slots(n) - 1u;
  p.filter = reinterpret_cast<uint32_t *>(reinterpret_cast<char *>(workspace) + (size_t)pairs_slots(n) * 16);
  p.filter_mask = pairs_slots(n) - 1u;
  p.kx = ksize[2];
  p.center_k = -1;
  for (int k = 0; k < (int)kv; ++k)
    if (p.off[k][0] == 0 && p.off[k][1] == 0 && p.off[k][2] == 0) p.center_k = k;
  hipError_t e = launch_subm_pairs(p, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "pair table launch");
  return CUMM_HIP_OK;
}

static size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

size_t cumm_hip_sort_by_mask_workspace(int n) { return sort_by_mask_workspace_bytes(n); }

int cumm_hip_sort_by_mask(const uint32_t *mask, int n, uint32_t mask_filter, uint32_t *sorted_mask,
                          int32_t *argsort, void *workspace, size_t workspace_bytes, void *stream) {
  return cumm_hip_sort_by_mask_ordered(mask, n, mask_filter, 0, sorted_mask, argsort, workspace, workspace_bytes, stream);
}

int cumm_hip_sort_by_mask_ordered(const uint32_t *mask, int n, uint32_t mask_filter, int order, uint32_t *sorted_mask,
                                  int32_t *argsort, void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || order < 0 || order > 1) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (order == 1 && (mask_filter >> 27) != 0u)
    return fail(CUMM_HIP_EINVAL, "the order by offset count takes filters of at most 27 bits (kernel volumes up to 27)");
  if (n == 0) return CUMM_HIP_OK;
  if (n >= (1 << 30)) return fail(CUMM_HIP_EINVAL, "too many positions");
  if (!mask || !sorted_mask || !argsort) return fail(CUMM_HIP_EINVAL, "mask, sorted_mask and argsort must not be empty");
  if (mask == sorted_mask) return fail(CUMM_HIP_EINVAL, "the sort is not in place: mask and sorted_mask must differ");
  if (!workspace || workspace_bytes < cumm_hip_sort_by_mask_workspace(n))
    return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", cumm_hip_sort_by_mask_workspace(n));
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(CUMM_HIP_EINVAL, "workspace must be 256-byte aligned");
  int32_t *status = nullptr;
  if (int rc = async_status_ptr(&status)) return rc;
  hipError_t e = launch_sort_by_mask(mask, n, mask_filter, sorted_mask, argsort, workspace, status + 1,
                                     light_hint_slot_ptr(sorted_mask), order, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "mask sort launch");
  return CUMM_HIP_OK;
}

int cumm_hip_light_prefix(const uint32_t *sorted_mask, int n, uint32_t mask_filter, int32_t *prefix, void *stream) {
  if (n < 0 || (n > 0 && !sorted_mask)) return fail(CUMM_HIP_EINVAL, "bad arguments");
  hipError_t e = launch_light_prefix(sorted_mask, n, mask_filter, prefix, n > 0 ? light_hint_slot_ptr(sorted_mask) : nullptr,
                                     reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "light prefix launch");
  return CUMM_HIP_OK;
}

int cumm_hip_query_light_hint(const uint32_t *sorted_mask, int n, uint32_t mask_filter, int32_t *prefix, int32_t *heavy_from,
                              void *stream) {
  if (!prefix) return fail(CUMM_HIP_EINVAL, "null out-param");
  *prefix = -1;
  if (heavy_from) *heavy_from = -1;
  if (!sorted_mask || n <= 0) return CUMM_HIP_OK;
  const int32_t *slot = light_hint_slot_ptr(sorted_mask);
  if (!slot) return CUMM_HIP_OK;
  int32_t words[8] = {};
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  HIP_TRY(hipMemcpyAsync(words, slot, sizeof(words), hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  const uint64_t key = (uint64_t)(uint32_t)words[0] | ((uint64_t)(uint32_t)words[1] << 32);
  if (key == (uint64_t)reinterpret_cast<uintptr_t>(sorted_mask) && words[2] == n && (uint32_t)words[3] == mask_filter)
  {
    *prefix = words[4];
    if (heavy_from) *heavy_from = words[5];
  }
  return CUMM_HIP_OK;
}

// ---- regular (strided) sparse convolution
namespace {
struct ConvPairsLayout {
  bool bitmap;         // small output grid: bitmap + prefix sums instead of hash set + sort
  unsigned long long n_words;
  uint32_t slots;
  size_t bound;        // most output sites n_in inputs can reach
  size_t off_uniq, off_sorted, off_counters, off_prefix, off_temp, total;
};
int gcd_int(int a, int b) { return b == 0 ? a : gcd_int(b, a % b); }
// out_shape as ConvProblem.calc_output_dims (cumm/conv/params.py:268-292 of the reference)
const char *conv_pairs_check(int batch_size, const int32_t *spatial_shape, const int32_t *ksize, const int32_t *stride,
                             const int32_t *padding, const int32_t *dilation, int32_t *out_shape,
                             unsigned long long *sites) {
  if (!spatial_shape || !ksize || !stride || !padding || !dilation) return "geometry arrays must not be empty";
  if (batch_size < 1) return "batch_size must be positive";
  const int64_t kv = (int64_t)ksize[0] * ksize[1] * ksize[2];
  if (ksize[0] < 1 || ksize[1] < 1 || ksize[2] < 1 || kv > kMaxKernelVolume) return "kernel volume must be 1..128";
  unsigned long long total = (unsigned long long)batch_size;
  for (int d = 0; d < 3; ++d) {
    if (spatial_shape[d] < 1 || dilation[d] < 1 || stride[d] < 1 || padding[d] < 0)
      return "spatial_shape, stride and dilation must be positive, padding not negative";
    const int64_t span = (int64_t)spatial_shape[d] + 2 * (int64_t)padding[d] - (int64_t)dilation[d] * (ksize[d] - 1) - 1;
    const int64_t o = span < 0 ? 0 : span / stride[d] + 1;
    if (o < 1 || o > (1 << 30)) return "empty output shape";
    out_shape[d] = (int32_t)o;
    if (total > (1ull << 62) / (unsigned long long)o) return "output grid of more than 2^62 sites";
    total *= (unsigned long long)o;
  }
  *sites = total;
  return nullptr;
}
// An input reaches, per axis, the offsets k with (x + pad - k*dilation) % stride == 0: every
// stride / gcd(stride, dilation)-th one.
bool conv_pairs_layout(int n_in, unsigned long long sites, const int32_t *ksize, const int32_t *stride,
                       const int32_t *dilation, ConvPairsLayout *l) {
  std::memset(l, 0, sizeof(*l));
  l->bitmap = sites <= (1ull << 33);
  if (l->bitmap) {
    l->n_words = ((sites + 31ull) / 32ull + 3ull) & ~3ull;
    l->off_prefix = align256((size_t)l->n_words * 4);
    l->off_temp = l->off_prefix + align256((size_t)l->n_words * 4 + 4);   // (+ the total)
    l->total = l->off_temp + align256(conv_pairs_scan_temp_bytes((size_t)l->n_words));
    return true;
  }
  int64_t per_input = 1;
  for (int d = 0; d < 3; ++d) {
    const int period = stride[d] / gcd_int(stride[d], dilation[d]);
    per_input *= (ksize[d] + period - 1) / period;
  }
  const int64_t bound = per_input * (int64_t)(n_in > 0 ? n_in : 0);
  if (bound >= ((int64_t)1 << 30)) return false;
  uint32_t slots = 1024;
  while ((int64_t)slots < bound + bound / 2) slots <<= 1;   // load factor at most two thirds
  l->slots = slots;
  l->bound = (size_t)bound;
  l->off_uniq = align256((size_t)slots * 16);
  l->off_sorted = l->off_uniq + align256(l->bound * 8 + 8);
  l->off_counters = l->off_sorted + align256(l->bound * 8 + 8);
  l->off_temp = l->off_counters + 256;
  l->total = l->off_temp + align256(conv_pairs_sort_temp_bytes(l->bound));
  return true;
}
void conv_pairs_params(ConvPairsParams *p, const ConvPairsLayout &l, const int32_t *coords, int n_in, int batch_size,
                       const int32_t *out_shape, const int32_t *ksize, const int32_t *stride, const int32_t *padding,
                       const int32_t *dilation, void *workspace) {
  std::memset(p, 0, sizeof(*p));
  p->coords = coords; p->n_in = n_in; p->batch = batch_size;
  p->kv = ksize[0] * ksize[1] * ksize[2];
  for (int d = 0; d < 3; ++d) { p->out_shape[d] = out_shape[d]; p->stride[d] = stride[d]; p->pad[d] = padding[d]; }
  for (int k = 0; k < p->kv; ++k) {
    p->koff[k][0] = (k / (ksize[1] * ksize[2])) * dilation[0];
    p->koff[k][1] = ((k / ksize[2]) % ksize[1]) * dilation[1];
    p->koff[k][2] = (k % ksize[2]) * dilation[2];
  }
  char *base = reinterpret_cast<char *>(workspace);
  if (l.bitmap) {
    p->bits = reinterpret_cast<uint32_t *>(base);
    p->prefix = reinterpret_cast<uint32_t *>(base + l.off_prefix);
    p->n_words = l.n_words;
    return;
  }
  p->table = base; p->slot_mask = l.slots - 1u;
  p->uniq = reinterpret_cast<unsigned long long *>(base + l.off_uniq);
  p->sorted = reinterpret_cast<unsigned long long *>(base + l.off_sorted);
  p->counters = reinterpret_cast<unsigned long long *>(base + l.off_counters);
}
}  // namespace

size_t cumm_hip_conv_pairs_workspace(int n_in, int batch_size, const int32_t *spatial_shape, const int32_t *ksize,
                                     const int32_t *stride, const int32_t *padding, const int32_t *dilation) {
  ConvPairsLayout l;
  int32_t out_shape[3];
  unsigned long long sites = 0;
  if (n_in < 0 || conv_pairs_check(batch_size, spatial_shape, ksize, stride, padding, dilation, out_shape, &sites)) return 0;
  if (!conv_pairs_layout(n_in, sites, ksize, stride, dilation, &l)) return 0;
  return l.total;
}

int cumm_hip_conv_pairs_sites(const int32_t *coords, int n_in, int batch_size, const int32_t *spatial_shape,
                              const int32_t *ksize, const int32_t *stride, const int32_t *padding,
                              const int32_t *dilation, int32_t *out_shape, int32_t *n_out, void *workspace,
                              size_t workspace_bytes, void *stream) {
  if (n_in < 0 || !out_shape || !n_out) return fail(CUMM_HIP_EINVAL, "bad arguments");
  unsigned long long sites = 0;
  if (const char *why = conv_pairs_check(batch_size, spatial_shape, ksize, stride, padding, dilation, out_shape, &sites))
    return fail(CUMM_HIP_EINVAL, "%s", why);
  *n_out = 0;
  if (n_in == 0) return CUMM_HIP_OK;
  ConvPairsLayout l;
  if (!conv_pairs_layout(n_in, sites, ksize, stride, dilation, &l)) return fail(CUMM_HIP_EINVAL, "too many voxels");
  if (!coords || !aligned16(coords)) return fail(CUMM_HIP_EINVAL, "coords must be 16-byte aligned and not empty");
  if (!workspace || workspace_bytes < l.total) return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", l.total);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(CUMM_HIP_EINVAL, "workspace must be 256-byte aligned");
  ConvPairsParams p;
  conv_pairs_params(&p, l, coords, n_in, batch_size, out_shape, ksize, stride, padding, dilation, workspace);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  char *temp = reinterpret_cast<char *>(workspace) + l.off_temp;
  // Either way the caller sizes its tables by the number of sites: the one synchronisation of the path.
  if (l.bitmap) {
    hipError_t e = launch_conv_pairs_bits(p, temp, l.total - l.off_temp, s);
    if (e != hipSuccess) return hip_fail(e, "output site launch");
    uint32_t total = 0;
    HIP_TRY(hipMemcpyAsync(&total, p.prefix + l.n_words, 4, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (total >= (1u << 31)) return fail(CUMM_HIP_ERUNTIME, "more than 2^31 output sites");
    *n_out = (int32_t)total;
    return CUMM_HIP_OK;
  }
  hipError_t e = launch_conv_pairs_sites(p, s);
  if (e != hipSuccess) return hip_fail(e, "output site launch");
  unsigned long long counters[2] = {0, 0};
  HIP_TRY(hipMemcpyAsync(counters, p.counters, sizeof(counters), hipMemcpyDeviceToHost, s));
  HIP_TRY(hipStreamSynchronize(s));
  if (counters[0] > l.bound) return fail(CUMM_HIP_ERUNTIME, "more output sites than the geometry allows (duplicate coordinates?)");
  p.n_out = (int)counters[0];
  int32_t *status = nullptr;
  if (int rc = async_status_ptr(&status)) return rc;
  e = launch_conv_pairs_sort(p, counters[1], temp, l.total - l.off_temp, status + 1, s);
  if (e != hipSuccess) return hip_fail(e, "output site sort");
  *n_out = p.n_out;
  return CUMM_HIP_OK;
}

int cumm_hip_conv_pairs_fill(const int32_t *coords, int n_in, int batch_size, const int32_t *spatial_shape,
                             const int32_t *ksize, const int32_t *stride, const int32_t *padding,
                             const int32_t *dilation, int n_out, int32_t *out_coords, int32_t *indices_fwd,
                             int32_t *indices_bwd, uint32_t *mask_fwd, uint32_t *mask_bwd, void *workspace,
                             size_t workspace_bytes, void *stream) {
  if (n_in < 0 || n_out < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  int32_t out_shape[3];
  unsigned long long sites = 0;
  if (const char *why = conv_pairs_check(batch_size, spatial_shape, ksize, stride, padding, dilation, out_shape, &sites))
    return fail(CUMM_HIP_EINVAL, "%s", why);
  if (n_in == 0) return CUMM_HIP_OK;
  ConvPairsLayout l;
  if (!conv_pairs_layout(n_in, sites, ksize, stride, dilation, &l)) return fail(CUMM_HIP_EINVAL, "too many voxels");
  if (!l.bitmap && (size_t)n_out > l.bound) return fail(CUMM_HIP_EINVAL, "n_out is not what cumm_hip_conv_pairs_sites returned");
  if (!coords || !aligned16(coords)) return fail(CUMM_HIP_EINVAL, "coords must be 16-byte aligned and not empty");
  if (n_out > 0 && (!out_coords || !indices_fwd || !aligned16(out_coords) || !aligned16(indices_fwd)))
    return fail(CUMM_HIP_EINVAL, "out_coords and indices_fwd (both 16-byte aligned) must not be empty");
  if ((int64_t)ksize[0] * ksize[1] * ksize[2] > 32 && (mask_fwd || mask_bwd))
    return fail(CUMM_HIP_EINVAL, "kernel volumes above 32 have no 32-bit masks: pass NULL for mask_fwd and mask_bwd");
  if (!workspace || workspace_bytes < l.total) return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", l.total);
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(CUMM_HIP_EINVAL, "workspace must be 256-byte aligned");
  ConvPairsParams p;
  conv_pairs_params(&p, l, coords, n_in, batch_size, out_shape, ksize, stride, padding, dilation, workspace);
  p.n_out = n_out;
  p.out_coords = out_coords; p.ind_f = indices_fwd; p.ind_b = indices_bwd; p.mask_f = mask_fwd; p.mask_b = mask_bwd;
  hipError_t e = launch_conv_pairs_fill(p, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "pair table launch");
  return CUMM_HIP_OK;
}

// ---- per-offset pair lists for the native (per-offset) convolution
size_t cumm_hip_pair_lists_workspace(int kv, int n) {
  if (kv <= 0 || n <= 0) return 0;
  const size_t chunks = ((size_t)n + kPairListChunk - 1) / kPairListChunk;
  return sizeof(int32_t) * (size_t)kv * chunks;
}

int cumm_hip_pair_lists(const int32_t *indices, int kv, int n, int32_t *pair_in, int32_t *pair_out, int32_t *counts,
                        void *workspace, size_t workspace_bytes, void *stream) {
  if (kv < 0 || n < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (kv == 0) return CUMM_HIP_OK;
  if (!counts) return fail(CUMM_HIP_EINVAL, "counts must not be empty");
  if (n > 0 && (!indices || !pair_in || !pair_out)) return fail(CUMM_HIP_EINVAL, "indices, pair_in and pair_out must not be empty");
  const size_t need = cumm_hip_pair_lists_workspace(kv, n);
  if (need > 0 && (!workspace || workspace_bytes < need)) return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", need);
  if (reinterpret_cast<uintptr_t>(workspace) & 3u) return fail(CUMM_HIP_EINVAL, "workspace must be 4-byte aligned");
  PairListsParams p;
  std::memset(&p, 0, sizeof(p));
  p.indices = indices; p.pair_in = pair_in; p.pair_out = pair_out; p.counts = counts;
  p.chunk_counts = reinterpret_cast<int32_t *>(workspace);
  p.kv = kv; p.n = n; p.chunks = (n + kPairListChunk - 1) / kPairListChunk;
  hipError_t e = launch_pair_lists(p, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "pair list launch");
  return CUMM_HIP_OK;
}

int cumm_hip_masks_from_pairs(const int32_t *indices, int kv, int n, uint32_t *mask, void *stream) {
  if (kv < 0 || n < 0 || kv > kMaxKernelVolume) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (kv == 0 || n == 0) return CUMM_HIP_OK;
  if (!indices || !mask) return fail(CUMM_HIP_EINVAL, "indices and mask must not be empty");
  hipError_t e = launch_masks_from_pairs(indices, mask, kv, n, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "mask launch");
  return CUMM_HIP_OK;
}

size_t cumm_hip_sort_by_mask_words_workspace(int n) {
  const size_t nn = (size_t)(n > 0 ? n : 1);
  return 2 * ((4 * nn + 255) & ~(size_t)255) + cumm_hip_sort_by_mask_workspace(n);
}

int cumm_hip_sort_by_mask_words(const uint32_t *mask, int n, int words, uint32_t *sorted_mask, int32_t *argsort,
                                void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || words < 1 || words > 4) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (n == 0) return CUMM_HIP_OK;
  if (n >= (1 << 30)) return fail(CUMM_HIP_EINVAL, "too many positions");
  if (!mask || !sorted_mask || !argsort) return fail(CUMM_HIP_EINVAL, "mask, sorted_mask and argsort must not be empty");
  if (mask == sorted_mask) return fail(CUMM_HIP_EINVAL, "the sort is not in place: mask and sorted_mask must differ");
  if (!workspace || workspace_bytes < cumm_hip_sort_by_mask_words_workspace(n))
    return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", cumm_hip_sort_by_mask_words_workspace(n));
  if (reinterpret_cast<uintptr_t>(workspace) & 255u) return fail(CUMM_HIP_EINVAL, "workspace must be 256-byte aligned");
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const size_t part = (4 * (size_t)n + 255) & ~(size_t)255;
  char *base = reinterpret_cast<char *>(workspace);
  uint32_t *keys = reinterpret_cast<uint32_t *>(base), *sorted_keys = reinterpret_cast<uint32_t *>(base + part);
  int32_t *status = nullptr;
  if (int rc = async_status_ptr(&status)) return rc;
  hipError_t e = launch_mask_words_keys(mask, keys, n, words, s);
  if (e == hipSuccess) e = launch_sort_by_mask(keys, n, 0xFFFFFFFFu, sorted_keys, argsort, base + 2 * part, status + 1, nullptr, 0, s);
  if (e == hipSuccess) e = launch_mask_words_gather(mask, argsort, sorted_mask, n, words, s);
  if (e != hipSuccess) return hip_fail(e, "mask sort launch");
  return CUMM_HIP_OK;
}

int cumm_hip_pairs_by_position(const int32_t *indices, const int32_t *mask_argsort, int kv, int n, int32_t *out,
                               void *stream) {
  if (kv < 0 || n < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (kv == 0 || n == 0) return CUMM_HIP_OK;
  if (!indices || !mask_argsort || !out) return fail(CUMM_HIP_EINVAL, "indices, mask_argsort and out must not be empty");
  if (out == indices) return fail(CUMM_HIP_EINVAL, "out must not be the table itself");
  hipError_t e = launch_pairs_by_position(indices, mask_argsort, out, kv, n, n, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "pair table permutation launch");
  return CUMM_HIP_OK;
}

// ---- stand-alone gather / scatter-add
namespace {
bool row_move_params(RowMoveParams *p, void *dst, const void *src, const int32_t *indices, int m, int rows_other,
                     size_t row_bytes, bool *wide) {
  *wide = row_bytes % 16 == 0 && aligned16(dst) && aligned16(src);
  const size_t piece = *wide ? 16 : 4;
  if (row_bytes / piece > 0xffffffffull) return false;
  p->src = src; p->dst = dst; p->indices = indices;
  p->per_row = (uint32_t)(row_bytes / piece);
  p->pieces = (uint64_t)m * p->per_row;
  p->shift = -1;
  for (int b = 0; b < 32; ++b)
    if (p->per_row == (1u << b)) p->shift = b;
  p->rows_other = rows_other;
  return true;
}
}  // namespace

int cumm_hip_gather_rows(void *output, const void *input, const int32_t *indices, int m, int rows_in,
                         size_t row_bytes, void *stream) {
  if (m < 0 || rows_in < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (row_bytes % 4) return fail(CUMM_HIP_ERUNTIME, "not supported. use supported() to check first");
  if (m == 0 || row_bytes == 0) return CUMM_HIP_OK;
  if (!output || !indices || (!input && rows_in > 0)) return fail(CUMM_HIP_EINVAL, "output, input and indices must not be empty");
  if ((reinterpret_cast<uintptr_t>(output) | reinterpret_cast<uintptr_t>(input)) & 3u)
    return fail(CUMM_HIP_EINVAL, "tensors must be 4-byte aligned");
  RowMoveParams p;
  bool wide = false;
  if (!row_move_params(&p, output, input, indices, m, rows_in, row_bytes, &wide)) return fail(CUMM_HIP_EINVAL, "rows too long");
  hipError_t e = launch_gather_rows(p, wide, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "gather launch");
  return CUMM_HIP_OK;
}

int cumm_hip_scatter_add_rows(void *output, const void *input, const int32_t *indices, int m, int rows_out,
                              int channels, int dtype, void *stream) {
  if (m < 0 || rows_out < 0 || channels < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (dtype != CUMM_HIP_F32 && dtype != CUMM_HIP_F16 && dtype != CUMM_HIP_BF16)
    return fail(CUMM_HIP_ERUNTIME, "can't find a suitable scatter: dtype must be f32, f16 or bf16");
  const size_t row_bytes = (size_t)channels * (dtype == CUMM_HIP_F32 ? 4 : 2);
  if (row_bytes % 4) return fail(CUMM_HIP_ERUNTIME, "not supported. use supported() to check first");
  if (m == 0 || row_bytes == 0 || rows_out == 0) return CUMM_HIP_OK;
  if (!output || !input || !indices) return fail(CUMM_HIP_EINVAL, "output, input and indices must not be empty");
  if ((reinterpret_cast<uintptr_t>(output) | reinterpret_cast<uintptr_t>(input)) & 3u)
    return fail(CUMM_HIP_EINVAL, "tensors must be 4-byte aligned");
  RowMoveParams p;
  bool wide = false;
  if (!row_move_params(&p, output, input, indices, m, rows_out, row_bytes, &wide)) return fail(CUMM_HIP_EINVAL, "rows too long");
  hipError_t e = launch_scatter_add_rows(p, dtype, wide, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "scatter launch");
  return CUMM_HIP_OK;
}

// ---- row-wise helpers
int cumm_hip_finish_rows(void *out, int dtype, const float *acc, const void *bias, int64_t rows, int channels,
                         float alpha, float beta, int act_type, float act_alpha, void *stream) {
  if (rows < 0 || channels < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (!is_float16_like(dtype)) return fail(CUMM_HIP_EINVAL, "the output must be f16 or bf16");
  if (channels % 8) return fail(CUMM_HIP_EINVAL, "channels must be a multiple of 8");
  if (rows == 0 || channels == 0) return CUMM_HIP_OK;
  if (!out || !acc || !aligned16(out) || !aligned16(acc) || (bias && !aligned16(bias)))
    return fail(CUMM_HIP_EINVAL, "out, acc (and bias) must be 16-byte aligned and not empty");
  FinishRowsParams p;
  std::memset(&p, 0, sizeof(p));
  p.out = out; p.acc = acc; p.bias = bias; p.rows = rows; p.channels = channels;
  p.alpha = alpha; p.beta = beta; p.act = act_type; p.act_alpha = act_alpha;
  hipError_t e = launch_finish_rows(p, dtype == CUMM_HIP_BF16, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "finish_rows launch");
  return CUMM_HIP_OK;
}

int cumm_hip_relu_backward(void *dst, const void *grad, const void *out, size_t elems, int dtype, void *stream) {
  if (!is_float16_like(dtype)) return fail(CUMM_HIP_EINVAL, "dtype must be f16 or bf16");
  if (elems % 8) return fail(CUMM_HIP_EINVAL, "the element count must be a multiple of 8");
  if (elems == 0) return CUMM_HIP_OK;
  if (!dst || !grad || !out || !aligned16(dst) || !aligned16(grad) || !aligned16(out))
    return fail(CUMM_HIP_EINVAL, "dst, grad and out must be 16-byte aligned and not empty");
  hipError_t e = launch_relu_backward(dst, grad, out, elems / 8, dtype == CUMM_HIP_BF16, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "relu_backward launch");
  return CUMM_HIP_OK;
}

size_t cumm_hip_column_sum_workspace(int64_t rows, int channels) {
  if (rows < 0 || channels <= 0) return 0;
  // (no rows: the sums are zeros, written through one block of partial sums all the same)
  return sizeof(float) * (size_t)column_sum_blocks(rows, channels) * (size_t)channels;
}

int cumm_hip_column_sum(void *dst, const void *src, int64_t rows, int channels, int dtype, void *workspace,
                        size_t workspace_bytes, void *stream) {
  if (rows < 0 || channels < 0) return fail(CUMM_HIP_EINVAL, "bad arguments");
  if (!is_float16_like(dtype)) return fail(CUMM_HIP_EINVAL, "dtype must be f16 or bf16");
  if (channels % 8 || channels > 2048) return fail(CUMM_HIP_EINVAL, "channels must be a multiple of 8, at most 2048");
  if (channels == 0) return CUMM_HIP_OK;
  if (!dst || (!src && rows > 0) || !aligned16(src)) return fail(CUMM_HIP_EINVAL, "dst and src (16-byte aligned) must not be empty");
  const size_t need = sizeof(float) * (size_t)column_sum_blocks(rows, channels) * (size_t)channels;
  if (!workspace || workspace_bytes < need) return fail(CUMM_HIP_ERUNTIME, "workspace at least %zu bytes.", need);
  if (reinterpret_cast<uintptr_t>(workspace) & 3u) return fail(CUMM_HIP_EINVAL, "workspace must be 4-byte aligned");
  ColumnSumParams p;
  std::memset(&p, 0, sizeof(p));
  p.dst = dst; p.src = src; p.partial = reinterpret_cast<float *>(workspace); p.rows = rows; p.channels = channels;
  hipError_t e = launch_column_sum(p, dtype == CUMM_HIP_BF16, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "column_sum launch");
  return CUMM_HIP_OK;
}

int cumm_hip_copy_kernel(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes % 16 || !aligned16(dst) || !aligned16(src)) return fail(CUMM_HIP_EINVAL, "copy needs 16-byte alignment");
  const size_t n = bytes / 16;
  if (n == 0) return CUMM_HIP_OK;
  size_t blocks = (n + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<v4i *>(dst), reinterpret_cast<const v4i *>(src), n);
  HIP_TRY(hipGetLastError());
  return CUMM_HIP_OK;
}

}  // extern "C"
