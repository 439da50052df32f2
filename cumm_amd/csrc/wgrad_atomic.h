// Backward-weight of the mask-based sparse convolution with work balanced over live tiles and
// fp32 atomic accumulation (the "split_k_parallel" flavour of the descriptor).
//
//   dW[:, r, :] = sum over sorted positions pos of  dOut[o]^T (x) In[indices[r][o]],  o = argsort[pos]
//
// The reference splits the positions into split_k_slices equal strides per kernel offset
// (cumm/conv/kernel.py:891-897, cumm/gemm/blockmma/mma.py:580-765): with sorted masks almost all
// work sits in one offset (the centre) and its slices serialise on a semaphore.  Here
//   * for its offset r every workgroup scans the reduced mask (one word per mask_width positions,
//     the forward's mask_output), counts the live tiles L_r and the offset gets ceil(L_r / QT)
//     workgroups, each taking an equal share of the LIVE tiles only; surplus workgroups exit;
//   * the workgroup first loads argsort and the pair-table entries of all its positions into LDS
//     (two memory round trips for everything), then streams 32 positions per step: gathered dOut
//     and In rows go to LDS transposed (contraction = positions must be contiguous for the MFMA),
//     the next step's rows are in flight while the current step computes;
//   * partial 64x64 blocks are added into an fp32 scratch image of dW with hardware float
//     atomics; a second kernel applies alpha/beta and converts to the weight type.
// The sum order is not fixed (fp32 atomics), the partial sums are never rounded to the weight type.
#pragma once
#include "common.h"

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
          __hip_atomic_fetch_add(p.scratch + mm * ldn + (int64_t)r * p.C + nn, acc[i][j][x],
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
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
};

// dW = cvt(alpha * scratch + beta * src) for the offsets enabled in mask_filter
template <class T>
__global__ __launch_bounds__(256) void wgrad_finalize_kernel(const WgradFinalizeParams p) {
  using E = Elem<T>;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= p.total) return;
  const int r = (int)((i / p.C) % p.kv);
  if (!((p.mask_filter >> r) & 1u)) return;
  uint16_t *dw = reinterpret_cast<uint16_t *>(p.dw);
  const uint16_t *src = reinterpret_cast<const uint16_t *>(p.src);
  float t = p.beta != 0.0f ? __builtin_fmaf(p.alpha, p.scratch[i], p.beta * E::to_float(src[i]))
                           : p.alpha * p.scratch[i];
  dw[i] = E::from_float(t);
}

}  // namespace cummhip
