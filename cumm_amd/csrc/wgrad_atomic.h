// Backward-weight of the mask-based sparse convolution with work balanced over live tiles and
// fp32 atomic accumulation (the "split_k_parallel" flavour of the descriptor).
//
//   dW[:, r, :] = sum over sorted positions pos of  dOut[o]^T (x) In[indices[r][o]],  o = argsort[pos]
//
// The reference splits the positions into split_k_slices equal strides per kernel offset
// (cumm/conv/kernel.py:891-897, cumm/gemm/blockmma/mma.py:580-765): with sorted masks almost all
// work sits in one offset (the centre) and its slices serialise on a semaphore.  Here the work of
// offset r is its LIVE tiles only (reduced mask word, i.e. the forward's mask_output, has bit r),
// cut into units of QT tiles; a unit makes one partial 64x64 block (per channel block) and adds
// it into an fp32 scratch image of dW with hardware float atomics; a last kernel applies
// alpha/beta and converts to the weight type.  Two ways to get there:
//   * wgrad_prepare_kernel + wgrad_units_kernel (workspace has room for the live-tile lists): the
//     prepare kernel compacts, per offset, the numbers of its live tiles and zeroes the images;
//     the unit kernel is a grid of resident workgroups that walk the units of all offsets.  A unit
//     resolves tile list -> argsort -> pair table for all of its positions at once, packs the
//     positions that have a pair, and streams their gathered rows through an LDS ring filled by
//     direct-to-LDS loads; the MFMA operands (contraction = pairs) come out of the row-major
//     tiles through transposing LDS reads.
//   * wgrad_atomic_kernel (no room for lists; image zeroed by a memset): a (groups, offsets) grid,
//     every workgroup scans the reduced mask for its offset itself and surplus workgroups exit;
//     rows pass through registers and are parked in LDS transposed with 16-bit stores.
// The sum order is not fixed (fp32 atomics), the partial sums are never rounded to the weight type.
//   * fixed-order variant (wgrad_units_kernel<..., true> + wgrad_finalize_ordered_kernel): the same
//     units, but a workgroup walks a contiguous run of them, carries its accumulator from unit to
//     unit of one (offset, channel block) and stores it into a slot of its own; the last kernel adds
//     the slots of an element in workgroup order.  Same bits from run to run on one device.
#pragma once
#include "common.h"
#include "lds_dma.h"

namespace cummhip {

struct WgradParams {
  const void *dout;   // [rows_y, K]
  const void *inp;    // [rows_x, C]
  float *scratch;     // [K, kv * C] fp32, zero on entry
  const int32_t *argsort;
  const int32_t *indices;   // [kv, n_idx]
  const uint32_t *red_mask; // [num_red]
  int32_t num_red, mask_width;
  uint32_t mask_filter;
  int32_t n_pos, n_idx, rows_x, rows_y;
  int32_t K, C, kv;
  int32_t tiles_per_wg;     // QT
  // live-tile lists made by wgrad_prepare_kernel (NULL: every workgroup scans the mask itself):
  // live_cnt[r] = number of tiles whose reduced mask has bit r, live_list[r * num_red + i] = the i-th
  const int32_t *live_cnt;
  const int32_t *live_list;
  // the unit-walking kernel spreads its atomics over `images` copies of the fp32 image, each
  // image_floats apart; the finalize kernel sums them
  int32_t images;
  int64_t image_floats;
  // one unit walks all 64 x 64 channel blocks of its positions in turn (the pair lists are made
  // once) instead of one block per unit; set by the launcher when the units are many anyway
  int32_t merge_blocks;
  // fixed-order variant (wgrad_units_kernel<..., true>): workgroup b walks the units
  // [b * q, (b + 1) * q) of the order (offset, channel block, share), keeps one accumulator while
  // offset and channel block stay the same and stores it - plain stores, no atomics - into slot
  // b + key (key = offset * channel blocks + channel block) of `scratch`; key_range[key] = {first
  // workgroup, number of workgroups} tells wgrad_finalize_ordered_kernel which slots to sum.
  int32_t *key_range;
};

constexpr int kWgradMaxPos = 1024;  // positions one workgroup handles at most (QT * mask_width)

template <class T>
__global__ __launch_bounds__(256) void wgrad_atomic_kernel(const WgradParams p) {
  using E = Elem<T>;
  constexpr int TK = 32, PV = 8, PITCH = TK + PV;
  __shared__ __attribute__((aligned(16))) uint16_t lds_x[64 * PITCH];
  __shared__ __attribute__((aligned(16))) uint16_t lds_y[64 * PITCH];
  __shared__ int lds_o[kWgradMaxPos];
  __shared__ int lds_i[kWgradMaxPos];
  __shared__ int lds_cnt[256];
  __shared__ int lds_list[kWgradMaxPos / 32];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, q = lane >> 4;

  const int kblocks = (p.K + 63) / 64, cblocks = (p.C + 63) / 64;
  int by = blockIdx.y;
  const int cb = by % cblocks; by /= cblocks;
  const int kb = by % kblocks; by /= kblocks;
  const int r = by;
  if (!((p.mask_filter >> r) & 1u)) return;

  // ---- live tiles of offset r: per-thread counts over a contiguous share, then a block scan
  const int share = (p.num_red + 255) / 256;
  const int t0 = tid * share;
  int cnt = 0;
  for (int t = t0; t < t0 + share && t < p.num_red; ++t) cnt += (p.red_mask[t] >> r) & 1u;
  lds_cnt[tid] = cnt;
  __syncthreads();
  // inclusive scan (Hillis-Steele; 256 entries)
  for (int off = 1; off < 256; off <<= 1) {
    const int v = tid >= off ? lds_cnt[tid - off] : 0;
    __syncthreads();
    lds_cnt[tid] += v;
    __syncthreads();
  }
  const int live = lds_cnt[255];
  const int n_wg = (live + p.tiles_per_wg - 1) / p.tiles_per_wg;
  if ((int)blockIdx.x >= n_wg) return;
  const int lo = (int)(((int64_t)blockIdx.x * live) / n_wg);
  const int hi = (int)(((int64_t)(blockIdx.x + 1) * live) / n_wg);
  int rank = lds_cnt[tid] - cnt;  // exclusive prefix
  for (int t = t0; t < t0 + share && t < p.num_red; ++t) {
    if ((p.red_mask[t] >> r) & 1u) {
      if (rank >= lo && rank < hi) lds_list[rank - lo] = t;
      ++rank;
    }
  }
  __syncthreads();
  const int n_list = hi - lo;
  const int mw = p.mask_width;
  const int n_slots = n_list * mw;  // <= kWgradMaxPos (checked on the host)

  // ---- argsort and pair-table entries of every position of this workgroup
  for (int s = tid; s < n_slots; s += 256) {
    const int pos = lds_list[s / mw] * mw + s % mw;
    int o = -1;
    if (pos < p.n_pos) o = p.argsort[pos];
    if (o >= p.rows_y) o = -1;
    lds_o[s] = o;
  }
  __syncthreads();
  for (int s = tid; s < n_slots; s += 256) {
    const int o = lds_o[s];
    int i = -1;
    if (o >= 0 && o < p.n_idx) i = p.indices[(int64_t)r * p.n_idx + o];
    if (i >= p.rows_x) i = -1;
    lds_i[s] = i;
    if (i < 0) lds_o[s] = -1;  // a position without a pair contributes nothing
  }
  __syncthreads();

  // ---- stream the positions, 32 per step
  const int kl = tid & 31, piece = tid >> 5;   // position inside the step, 8-channel piece
  const int ych = kb * 64 + piece * 8, xch = cb * 64 + piece * 8;
  const char *yb = reinterpret_cast<const char *>(p.dout);
  const char *xb = reinterpret_cast<const char *>(p.inp);
  auto load_rows = [&](int step, v4i &yv, v4i &xv) {
    const int o = lds_o[step * TK + kl], i = lds_i[step * TK + kl];
    yv = v4i{0, 0, 0, 0};
    xv = v4i{0, 0, 0, 0};
    if (o >= 0) {
      if (ych < p.K) yv = *reinterpret_cast<const v4i *>(yb + ((int64_t)o * p.K + ych) * 2);
      if (xch < p.C) xv = *reinterpret_cast<const v4i *>(xb + ((int64_t)i * p.C + xch) * 2);
    }
  };
  auto park_rows = [&](const v4i &yv, const v4i &xv) {
    const uint16_t *ys = reinterpret_cast<const uint16_t *>(&yv);
    const uint16_t *xs = reinterpret_cast<const uint16_t *>(&xv);
#pragma unroll
    for (int e = 0; e < PV; ++e) {
      lds_y[(piece * PV + e) * PITCH + kl] = ys[e];
      lds_x[(piece * PV + e) * PITCH + kl] = xs[e];
    }
  };

  v4f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = v4f{0, 0, 0, 0};

  auto compute = [&]() {
    v4i xf[2], yf[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
      xf[j] = *reinterpret_cast<const v4i *>(&lds_x[((wn * 2 + j) * 16 + l16) * PITCH + q * PV]);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      yf[i] = *reinterpret_cast<const v4i *>(&lds_y[((wm * 2 + i) * 16 + l16) * PITCH + q * PV]);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = E::mfma(yf[i], xf[j], acc[i][j]);
  };

  const int n_steps = n_slots / TK;  // mask_width is a multiple of 32
  v4i ya, xa, yb2, xb2;
  if (n_steps > 0) load_rows(0, ya, xa);
  for (int s = 0; s < n_steps; s += 2) {
    // two steps per trip so that the register set being filled is never the one being parked
    if (s + 1 < n_steps) load_rows(s + 1, yb2, xb2);
    park_rows(ya, xa);
    __syncthreads();
    compute();
    __syncthreads();
    if (s + 1 < n_steps) {
      if (s + 2 < n_steps) load_rows(s + 2, ya, xa);
      park_rows(yb2, xb2);
      __syncthreads();
      compute();
      __syncthreads();
    }
  }

  // ---- add the partial block into the fp32 image.  dOut is the MFMA row operand, so a lane
  // holds K indices 4q + x and one C index l16: for a fixed x the 16 lanes of a quarter hit 16
  // consecutive floats (one 64-byte segment per quarter).
  const int64_t ldn = (int64_t)p.kv * p.C;
  float *image = p.scratch;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int nn = cb * 64 + (wn * 2 + j) * 16 + l16;
      if (nn >= p.C) continue;
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const int mm = kb * 64 + (wm * 2 + i) * 16 + 4 * q + x;
        if (mm < p.K)
          __hip_atomic_fetch_add(image + mm * ldn + (int64_t)r * p.C + nn, acc[i][j][x],
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

// ---- variant that reads the live-tile lists made by wgrad_prepare_kernel: a resident grid whose
// workgroups walk the units (offset r, channel blocks, share x of the offset's live tiles) u = b,
// b + G, ...: no workgroup scans the mask, none is launched only to find that it has nothing to do.
struct WgradPrepareParams {
  float *scratch;             // zeroed here
  int64_t scratch_floats;
  const uint32_t *red_mask;
  int32_t num_red, kv;
  uint32_t mask_filter;
  int32_t *live_cnt;          // [32]
  int32_t *live_list;         // [kv * num_red]
};

// workgroup r < kv compacts the tiles of offset r; the others zero the fp32 image
static __global__ __launch_bounds__(256) void wgrad_prepare_kernel(const WgradPrepareParams p) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if ((int)blockIdx.x >= p.kv) {
    const int64_t nz = (int64_t)(gridDim.x - p.kv) * 256;   // scratch_floats is a multiple of 4
    v4f *z = reinterpret_cast<v4f *>(p.scratch);
    for (int64_t i = (int64_t)(blockIdx.x - p.kv) * 256 + tid; i < p.scratch_floats / 4; i += nz) z[i] = v4f{0, 0, 0, 0};
    return;
  }
  __shared__ int wave_cnt[2][4];
  const int r = blockIdx.x;
  const bool on = (p.mask_filter >> r) & 1u;
  int base = 0;
  constexpr int U = 8;   // mask words a thread has in flight
  const v4i rs_red = rsrc_words(p.red_mask, (uint32_t)p.num_red * 4u);
  for (int t0 = 0; t0 < p.num_red; t0 += 256 * U) {
    // (hidden loads, one wait: as conditional loads each of the U got a branch and a wait)
    int m[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = t0 + u * 256 + tid;
      m[u] = load_b32_hidden(rs_red, t < p.num_red ? (uint32_t)t * 4u : 0x80000000u);
    }
    wait_vmcnt<0>();
#pragma unroll
    for (int u = 0; u < U; ++u) keep_after_wait(m[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = t0 + u * 256 + tid;
      const bool live = on && (((uint32_t)m[u] >> r) & 1u);
      const uint64_t bal = __ballot(live);
      if (lane == 0) wave_cnt[u & 1][wave] = __builtin_popcountll(bal);
      __syncthreads();   // the other set of counters is free again: everybody passed the previous barrier
      int before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int c = wave_cnt[u & 1][w];
        before += w < wave ? c : 0;
        total += c;
      }
      if (live) p.live_list[(int64_t)r * p.num_red + base + before + __builtin_popcountll(bal & ((1ull << lane) - 1ull))] = t;
      base += total;
    }
  }
  if (tid == 0) p.live_cnt[r] = base;
}

// a / b for 0 <= a < 2^22, 0 < b < 2^22, without the long integer-division sequence
__device__ __forceinline__ int fast_div(int a, int b) {
  int qn = (int)((float)a * __builtin_amdgcn_rcpf((float)b));
  const int rem = a - qn * b;
  if (rem < 0) --qn;
  if (rem >= b) ++qn;
  return qn;
}

// inclusive prefix sum over the 64 lanes of a wave with row shifts and row broadcasts
__device__ __forceinline__ int wave_prefix_sum_dpp(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, true);   // row_bcast:15 into rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, true);   // row_bcast:31 into rows 2, 3
  return v;
}

// KB, CB = 64-channel blocks of dOut (K) and of In (C) that a unit multiplies in one pass, H =
// 32-pair halves per step.  <1, 1, 2> is the unit described above.  <2, 2, 1> takes 128 x 128
// channels: the full 256-byte rows of a pair are gathered once instead of one 128-byte half per
// 64 x 64 block (four gathers of each pair at C = K = 128, where the launch is bound by that
// traffic once dOut and In no longer fit the last-level cache); its stage holds 32 pairs (16 KB,
// four stages, still two workgroups per CU) and a wave accumulates 64 x 64.
template <class T, int KB, int CB, int H, bool DET = false>
__global__ __launch_bounds__(256) void wgrad_units_kernel(const WgradParams p) {
  using E = Elem<T>;
  constexpr int TK = 32 * H;          // pairs per step
  constexpr int NS = 4, L = NS - 1;   // ring stages, steps the loads run ahead
  constexpr int PART = 4096;          // one tile: 32 rows x 128 bytes
  constexpr int HALF = (KB + CB) * PART;   // the dOut tiles, then the In tiles
  constexpr int STAGE = H * HALF;
  constexpr int MAXIT = kWgradMaxPos / 256;
  constexpr int NJ = 2 * KB, NI = 2 * CB;   // 16-channel blocks of dOut / In per wave
  __shared__ __attribute__((aligned(16))) char ring[NS * STAGE];
  __shared__ int lds_o[kWgradMaxPos + TK];
  __shared__ int lds_i[kWgradMaxPos + TK];
  __shared__ int wave_cnt[MAXIT][4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, q = lane >> 4;

  const int kblocks = (p.K + 64 * KB - 1) / (64 * KB), cblocks = (p.C + 64 * CB - 1) / (64 * CB);
  const int per_r = (!DET && p.merge_blocks) ? 1 : kblocks * cblocks;
  const int combos = (!DET && p.merge_blocks) ? kblocks * cblocks : 1;
  // units of offset r: its workgroups (ceil(live / QT)) times the channel blocks.  Lane r of every
  // wave holds offset r's numbers (kv <= 32: one mask bit per offset); a prefix sum over the
  // lanes and a ballot locate a unit without a loop over memory.
  const int my_live = lane < p.kv ? p.live_cnt[lane] : 0;
  const v4i rs_list = rsrc_words(p.live_list, (uint32_t)p.kv * (uint32_t)p.num_red * 4u);
  const v4i rs_sort = rsrc_words(p.argsort, (uint32_t)p.n_pos * 4u);
  const v4i rs_idx = rsrc_words(p.indices, (uint32_t)p.kv * (uint32_t)p.n_idx * 4u);
  const v4i y_rsrc = rsrc_words(p.dout, (uint32_t)p.rows_y * (uint32_t)p.K * 2u);
  const v4i x_rsrc = rsrc_words(p.inp, (uint32_t)p.rows_x * (uint32_t)p.C * 2u);
  const int mw = p.mask_width;

  // ---- what does not depend on the unit: which chunk of which row of a stage this lane fetches,
  // where this lane's transposing reads point
  const int srow = tid >> 3, schunk = tid & 7;
  auto swz = [](int row) { return 2 * ((row >> 1) & 3); };
  const uint32_t ring_at = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds_addr(ring) + wave * 1024));
  int y_rd[2][NJ], x_rd[2][NI];   // [4-row group h of a read pair][16-channel block of this wave]
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = q * 8 + h * 4 + (l16 >> 2);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int g = wm * NJ + j;   // 16-channel block among the unit's 4 * KB: tile g / 4, column block g % 4
      const int ycol = (g & 3) * 16 + 4 * (l16 & 3);
      y_rd[h][j] = (g >> 2) * PART + row * 128 + (((ycol >> 3) ^ swz(row)) * 16) + (ycol & 7) * 2;
    }
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int g = wn * NI + j;
      const int xcol = (g & 3) * 16 + 4 * (l16 & 3);
      x_rd[h][j] = (KB + (g >> 2)) * PART + row * 128 + (((xcol >> 3) ^ swz(row)) * 16) + (xcol & 7) * 2;
    }
  }

  // (the address arithmetic above runs while the counts are on their way)
  // Tiles per unit: as few as still leave every workgroup of the grid at most one unit - shorter
  // units end sooner, and the longest unit is the launch's critical path -, at most what the LDS
  // lists hold.  (Every offset may add a partly filled unit: kv * per_r workgroups are set aside.)
  int tiles_per_unit = p.tiles_per_wg;
  {
    const int total_live = __builtin_amdgcn_readlane(wave_prefix_sum_dpp(my_live), 31);
    const int room = (int)gridDim.x - p.kv * per_r;
    if (room > 0) {
      int fewest = fast_div(total_live * per_r + room - 1, room);
      fewest = fewest < 2 ? 2 : fewest;
      tiles_per_unit = fewest < tiles_per_unit ? fewest : tiles_per_unit;
    }
  }
  const int my_wgs = fast_div(my_live + tiles_per_unit - 1, tiles_per_unit);
  const int my_units = my_wgs * per_r;
  const int incl = wave_prefix_sum_dpp(my_units);
  const int total_units = __builtin_amdgcn_readlane(incl, 31);

  // fixed-order variant: a contiguous run of units per workgroup, and the table of the workgroups
  // that hold a partial sum of each (offset, channel block)
  const int run = DET ? (total_units + (int)gridDim.x - 1) / (int)gridDim.x : 1;
  if constexpr (DET) {
    if (blockIdx.x == 0) {
      __shared__ int key_wgs[32], key_start[32];
      if (tid < 32) {
        key_wgs[tid] = my_wgs;
        key_start[tid] = incl - my_units;
      }
      __syncthreads();
      for (int key = tid; key < p.kv * per_r; key += 256) {
        const int r = key / per_r, combo = key - r * per_r;
        const int n = key_wgs[r], first = key_start[r] + combo * n;
        p.key_range[2 * key] = n > 0 ? first / run : 0;
        p.key_range[2 * key + 1] = n > 0 ? (first + n - 1) / run - first / run + 1 : 0;
      }
    }
  }
  v4f acc[NJ][NI];
  int acc_key = -1;
  auto store_acc = [&]() __attribute__((always_inline)) {
    float *slot = p.scratch + (int64_t)((int)blockIdx.x + acc_key) * (64 * KB * 64 * CB);
#pragma unroll
    for (int i = 0; i < NJ; ++i)
#pragma unroll
      for (int j = 0; j < NI; ++j)
#pragma unroll
        for (int x = 0; x < 4; ++x)
          slot[((wm * NJ + i) * 16 + 4 * q + x) * (64 * CB) + (wn * NI + j) * 16 + l16] = acc[i][j][x];
  };
  const int unit_begin = DET ? (int)blockIdx.x * run : (int)blockIdx.x;
  const int unit_end = DET ? (unit_begin + run < total_units ? unit_begin + run : total_units) : total_units;
  const int unit_step = DET ? 1 : (int)gridDim.x;

  for (int unit = unit_begin; unit < unit_end; unit += unit_step) {
    const int r = __builtin_amdgcn_readfirstlane(__builtin_popcountll(__ballot(lane < 32 && incl <= unit)));
    const int u = unit - __builtin_amdgcn_readlane(incl - my_units, r);
    const int live = __builtin_amdgcn_readlane(my_live, r);
    const int n_wg = __builtin_amdgcn_readlane(my_wgs, r);
    int bx = u, cb = 0, kb = 0;
    if constexpr (DET) {
      // units of an offset in the order (channel block, share): a workgroup's run stays on one
      // accumulator for as long as possible
      const int combo = fast_div(u, n_wg);
      bx = u - combo * n_wg;
      kb = fast_div(combo, cblocks);
      cb = combo - kb * cblocks;
      const int key = r * per_r + combo;
      if (key != acc_key) {
        if (acc_key >= 0) store_acc();
        acc_key = key;
#pragma unroll
        for (int i = 0; i < NJ; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) acc[i][j] = v4f{0, 0, 0, 0};
      }
    } else if (per_r > 1) {
      bx = fast_div(u, per_r);
      const int rest = u - bx * per_r;
      kb = fast_div(rest, cblocks);
      cb = rest - kb * cblocks;
    }
    // equal shares of the live tiles: the first live % n_wg workgroups take one more
    const int share = fast_div(live, n_wg), extra = live - share * n_wg;
    const int lo = bx * share + (bx < extra ? bx : extra);
    const int n_list = share + (bx < extra ? 1 : 0);
    const int n_slots = n_list * mw;  // <= kWgradMaxPos (checked on the host)

    // ---- the (dOut row, In row) pairs of this unit's positions: tile list -> argsort -> pair
    // table, three dependent loads per position, all positions of the unit at once.  Each level
    // is issued for all positions as hidden buffer loads (a position past the end reads 0
    // through the descriptor and is sorted out with a select) and waited for once: as
    // conditional C++ loads every one of the twelve got a branch and a wait of its own.
    int t_[MAXIT], o_[MAXIT], i_[MAXIT], within[MAXIT];
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      const int s = k * 256 + tid;
      const int ti = fast_div(s, mw);
      within[k] = s - ti * mw;
      t_[k] = load_b32_hidden(rs_list, s < n_slots ? (uint32_t)(r * p.num_red + lo + ti) * 4u : 0x80000000u);
    }
    wait_vmcnt<0>();   // (also the previous unit's atomics)
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) keep_after_wait(t_[k]);
    bool have[MAXIT];
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      const int pos = t_[k] * mw + within[k];
      have[k] = k * 256 + tid < n_slots && pos < p.n_pos;
      o_[k] = load_b32_hidden(rs_sort, have[k] ? (uint32_t)pos * 4u : 0x80000000u);
    }
    wait_vmcnt<0>();
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) keep_after_wait(o_[k]);
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      const int o = o_[k];
      o_[k] = have[k] && o >= 0 && o < p.rows_y && o < p.n_idx ? o : -1;
      i_[k] = load_b32_hidden(rs_idx, o_[k] >= 0 ? (uint32_t)(r * p.n_idx + o_[k]) * 4u : 0x80000000u);
    }
    wait_vmcnt<0>();
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) keep_after_wait(i_[k]);
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) i_[k] = o_[k] >= 0 && i_[k] < p.rows_x ? i_[k] : -1;
    // Positions without a pair are dropped: the pairs are packed into the front of the LDS lists
    // (ballot + prefix counts), so that a sparse offset streams only the rows it has.
    uint64_t bal[MAXIT];
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      bal[k] = __ballot(i_[k] >= 0);
      if (lane == 0) wave_cnt[k][wave] = __builtin_popcountll(bal[k]);
    }
    __syncthreads();
    int n_pairs = 0;
#pragma unroll
    for (int k = 0; k < MAXIT; ++k) {
      int before = 0, total = 0;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int c = wave_cnt[k][w];
        before += w < wave ? c : 0;
        total += c;
      }
      if (i_[k] >= 0) {
        const int dst = n_pairs + before + __builtin_popcountll(bal[k] & ((1ull << lane) - 1ull));
        lds_o[dst] = o_[k];
        lds_i[dst] = i_[k];
      }
      n_pairs += total;
    }
    if (tid < TK) {   // the last step's empty slots
      lds_o[n_pairs + tid] = -1;
      lds_i[n_pairs + tid] = -1;
    }
    __syncthreads();
    const int n_steps = (n_pairs + TK - 1) / TK;

    // ---- stream the pairs, 64 per step, through a ring of NS stages.  Each 32-pair half of a
    // stage holds the gathered dOut and In rows as they are (row = pair, 128 bytes = this block's 64 channels,
    // 16-byte chunks XOR-permuted by 2*((row/2)%4) against bank conflicts), written by
    // direct-to-LDS loads: lane l of wave w fetches one 16-byte chunk of row 8w + l/8, so 8
    // neighbouring lanes read one row's 128 bytes and the permutation is applied by choosing
    // which chunk a lane fetches.  An empty slot, a channel past the end and a step past the end
    // are fetched at an offset outside the buffer: zeros arrive, no memory is touched, and the
    // number of loads in flight stays the same on every path (the waits below count
    // instructions).  The MFMA operands need 8 consecutive PAIRS of one channel per lane, i.e.
    // columns of these tiles: ds_read_b64_tr_b16 delivers them (lane s of a 16-lane group points
    // at row r0 + s/4, channels 4*(s%4)..; lane i receives rows r0 .. r0+3 of channel i).
    // Step s waits for its own stage, passes the barrier (everybody's loads of step s have
    // landed, everybody is done with step s-1), reads its operands, refills the stage of step
    // s-1 with step s+NS-1, computes.
    for (int combo = 0; combo < combos; ++combo) {
    if (p.merge_blocks) {
      kb = fast_div(combo, cblocks);
      cb = combo - kb * cblocks;
    }
    const int ych = kb * (64 * KB) + (schunk ^ swz(srow)) * 8, xch = cb * (64 * CB) + (schunk ^ swz(srow)) * 8;
    auto offsets = [&](int t, uint32_t (&yoff)[H][KB], uint32_t (&xoff)[H][CB]) __attribute__((always_inline)) {
#pragma unroll
      for (int hh = 0; hh < H; ++hh) {
#pragma unroll
        for (int pp = 0; pp < KB; ++pp) yoff[hh][pp] = 0x80000000u;
#pragma unroll
        for (int pp = 0; pp < CB; ++pp) xoff[hh][pp] = 0x80000000u;
        if (t < n_steps) {
          const int o = lds_o[t * TK + hh * 32 + srow], i = lds_i[t * TK + hh * 32 + srow];
          if (o >= 0) {
#pragma unroll
            for (int pp = 0; pp < KB; ++pp)
              if (ych + pp * 64 < p.K) yoff[hh][pp] = (uint32_t)(o * p.K + ych + pp * 64) * 2u;
#pragma unroll
            for (int pp = 0; pp < CB; ++pp)
              if (xch + pp * 64 < p.C) xoff[hh][pp] = (uint32_t)(i * p.C + xch + pp * 64) * 2u;
          }
        }
      }
    };
    auto issue = [&](int t, const uint32_t (&yoff)[H][KB], const uint32_t (&xoff)[H][CB]) __attribute__((always_inline)) {
      const uint32_t dst = ring_at + (uint32_t)__builtin_amdgcn_readfirstlane((t % NS) * STAGE);
#pragma unroll
      for (int hh = 0; hh < H; ++hh) {
#pragma unroll
        for (int pp = 0; pp < KB; ++pp) dma_b128(y_rsrc, dst + hh * HALF + pp * PART, yoff[hh][pp], 0);
#pragma unroll
        for (int pp = 0; pp < CB; ++pp) dma_b128(x_rsrc, dst + hh * HALF + (KB + pp) * PART, xoff[hh][pp], 0);
      }
    };

    if constexpr (!DET) {
#pragma unroll
      for (int i = 0; i < NJ; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = v4f{0, 0, 0, 0};
    }

    wait_vmcnt<0>();   // the previous unit's atomics: from here on the counter holds ring loads only
    uint32_t yn[H][KB], xn[H][CB];
    for (int t = 0; t < L; ++t) {
      offsets(t, yn, xn);
      issue(t, yn, xn);
    }
    offsets(L, yn, xn);
    for (int s = 0; s < n_steps; ++s) {
      wait_vmcnt<(KB + CB) * H * (L - 1)>();
      lds_barrier();
      typedef short v4s __attribute__((ext_vector_type(4)));
      typedef __attribute__((address_space(3))) v4s *lds_v4s;
      const char *base = ring + (s % NS) * STAGE;
      v4i xf[H][NI], yf[H][NJ];
#pragma unroll
      for (int hh = 0; hh < H; ++hh) {
        const char *hb = base + hh * HALF;
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const v4s ylo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)CUMM_LDS_PTR(hb + y_rd[0][j]));
          const v4s yhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)CUMM_LDS_PTR(hb + y_rd[1][j]));
          yf[hh][j] = __builtin_bit_cast(v4i, __builtin_shufflevector(ylo, yhi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          const v4s xlo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)CUMM_LDS_PTR(hb + x_rd[0][j]));
          const v4s xhi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)CUMM_LDS_PTR(hb + x_rd[1][j]));
          xf[hh][j] = __builtin_bit_cast(v4i, __builtin_shufflevector(xlo, xhi, 0, 1, 2, 3, 4, 5, 6, 7));
        }
      }
      issue(s + L, yn, xn);
      offsets(s + L + 1, yn, xn);
#pragma unroll
      for (int hh = 0; hh < H; ++hh)
#pragma unroll
        for (int i = 0; i < NJ; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j) acc[i][j] = E::mfma(yf[hh][i], xf[hh][j], acc[i][j]);
    }
    wait_vmcnt<0>();   // the fetches past the end

    // ---- add the partial block into an fp32 image.  dOut is the MFMA row operand, so a lane
    // holds K indices 4q + x and one C index l16: for a fixed x the 16 lanes of a quarter hit 16
    // consecutive floats (one 64-byte segment per quarter).  Units that follow each other go to
    // different images, so that the many units of one offset do not all queue on the same
    // addresses.
    if (!DET && n_steps > 0) {
      const int64_t ldn = (int64_t)p.kv * p.C;
      float *image = p.scratch + (int64_t)(unit % p.images) * p.image_floats;
#pragma unroll
      for (int i = 0; i < NJ; ++i) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          const int nn = cb * (64 * CB) + (wn * NI + j) * 16 + l16;
          if (nn >= p.C) continue;
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            const int mm = kb * (64 * KB) + (wm * NJ + i) * 16 + 4 * q + x;
            if (mm < p.K)
              __hip_atomic_fetch_add(image + mm * ldn + (int64_t)r * p.C + nn, acc[i][j][x],
                                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
    }
    lds_barrier();     // every wave is done with the ring before the next block's loads land in it
    }  // channel blocks
    __syncthreads();   // the LDS lists and the ring are rewritten by the next unit
  }
  if constexpr (DET) {
    if (acc_key >= 0) store_acc();
  }
}

struct WgradFinalizeParams {
  const float *scratch;
  void *dw;
  const void *src;
  int64_t total;   // K * kv * C
  int32_t C, kv;
  uint32_t mask_filter;
  float alpha, beta;
  int32_t images;  // copies of the image to sum (each `total` floats, rounded up to 64 floats, apart)
  int64_t image_floats;
};

// dW = cvt(alpha * sum of the scratch images + beta * src) for the offsets enabled in mask_filter
// Four consecutive elements per thread (C is a multiple of 8, so they share their offset).
template <class T>
__global__ __launch_bounds__(256) void wgrad_finalize_kernel(const WgradFinalizeParams p) {
  using E = Elem<T>;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= p.total) return;
  const int r = (int)((i / p.C) % p.kv);
  if (!((p.mask_filter >> r) & 1u)) return;
  // up to 8 images, all requested at once (a loop over p.images would wait for each): images
  // past the count are read at an offset outside the descriptor and arrive as zeros
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float *>(p.scratch), 0, (int)((uint32_t)p.images * (uint32_t)p.image_floats * 4u), 0x00020000);
  v4f part[8];
#pragma unroll
  for (int g = 0; g < 8; ++g)
    part[g] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
        rs, g < p.images ? (uint32_t)((int64_t)g * p.image_floats + i) * 4u : 0x80000000u, 0, 0));
  v4f acc = part[0];
#pragma unroll
  for (int g = 1; g < 8; ++g) acc += part[g];
  typedef uint16_t v4h __attribute__((ext_vector_type(4)));
  v4h out;
  if (p.beta != 0.0f) {
    const v4h src = *reinterpret_cast<const v4h *>(reinterpret_cast<const uint16_t *>(p.src) + i);
#pragma unroll
    for (int x = 0; x < 4; ++x) out[x] = E::from_float(__builtin_fmaf(p.alpha, acc[x], p.beta * E::to_float(src[x])));
  } else {
#pragma unroll
    for (int x = 0; x < 4; ++x) out[x] = E::from_float(p.alpha * acc[x]);
  }
  *reinterpret_cast<v4h *>(reinterpret_cast<uint16_t *>(p.dw) + i) = out;
}

// dW = cvt(alpha * (sum of the slots of an element's (offset, channel block), in workgroup order) +
// beta * src) for the fixed-order variant.  Eight lanes share four consecutive elements: lane g sums
// the g-th eighth of the slots first to last, then the eight sums are combined pairwise (1, 2, 4
// lanes apart): the shape of the sum depends on the number of slots only, so the result repeats bit
// for bit from run to run.
struct WgradOrderedParams {
  const float *slots;
  const int32_t *key_range;
  void *dw;
  const void *src;
  int64_t total;        // K * kv * C
  int32_t K, C, kv;
  int32_t block_k, block_c;   // channels of a slot (64 or 128 each)
  int32_t cblocks, per_r;
  uint32_t mask_filter;
  float alpha, beta;
  uint32_t slots_bytes;
};

template <class T>
__global__ __launch_bounds__(256) void wgrad_finalize_ordered_kernel(const WgradOrderedParams p) {
  using E = Elem<T>;
  const int g = threadIdx.x & 7;
  const int64_t i = ((int64_t)blockIdx.x * 32 + (threadIdx.x >> 3)) * 4;
  const bool in_range = i < p.total;
  const int64_t ii = in_range ? i : 0;
  const int nn = (int)(ii % p.C);
  const int r = (int)((ii / p.C) % p.kv);
  const int mm = (int)(ii / ((int64_t)p.C * p.kv));
  const bool on = in_range && ((p.mask_filter >> r) & 1u);
  const int kb = mm / p.block_k, cb = nn / p.block_c;
  const int key = r * p.per_r + kb * p.cblocks + cb;
  const int first = p.key_range[2 * key], count = on ? p.key_range[2 * key + 1] : 0;
  const int64_t slot_floats = (int64_t)p.block_k * p.block_c;
  const uint32_t within = (uint32_t)((mm - kb * p.block_k) * p.block_c + (nn - cb * p.block_c)) * 4u;
  const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.slots), 0, (int)p.slots_bytes, 0x00020000);
  const int share = (count + 7) >> 3;
  const int lo = g * share, hi = lo + share < count ? lo + share : count;
  v4f sum = v4f{0, 0, 0, 0};
  for (int t0 = lo; t0 < hi; t0 += 8) {
    v4f part[8];
#pragma unroll
    for (int u = 0; u < 8; ++u)
      part[u] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(
          rs, t0 + u < hi ? (uint32_t)((int64_t)(first + key + t0 + u) * slot_floats * 4) + within : 0x80000000u, 0, 0));
#pragma unroll
    for (int u = 0; u < 8; ++u) sum += part[u];   // (a slot past the share arrives as +0)
  }
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    float v = sum[x];
    v += __shfl_xor(v, 1, 64);
    v += __shfl_xor(v, 2, 64);
    v += __shfl_xor(v, 4, 64);
    sum[x] = v;
  }
  if (!on || g != 0) return;
  typedef uint16_t v4h __attribute__((ext_vector_type(4)));
  v4h out;
  if (p.beta != 0.0f) {
    const v4h src = *reinterpret_cast<const v4h *>(reinterpret_cast<const uint16_t *>(p.src) + i);
#pragma unroll
    for (int x = 0; x < 4; ++x) out[x] = E::from_float(__builtin_fmaf(p.alpha, sum[x], p.beta * E::to_float(src[x])));
  } else {
#pragma unroll
    for (int x = 0; x < 4; ++x) out[x] = E::from_float(p.alpha * sum[x]);
  }
  *reinterpret_cast<v4h *>(reinterpret_cast<uint16_t *>(p.dw) + i) = out;
}

}  // namespace cummhip
