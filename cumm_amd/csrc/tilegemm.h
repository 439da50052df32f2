// LDS-tiled MFMA GEMM for gfx950:  D[m][n] = epilogue( sum_k Y[m][k] * X[n][k] ).
//
// One kernel family covers the dense GEMM (all transpose combinations), the ShuffleAB GEMM
// (C = A[a_inds]^T B[b_inds]) and the mask-based sparse-convolution backward-weight pass
// (dW[:, r, :] = sum over positions of dOut[o]^T (x) In[indices[r][o]]), with serial split-K.
//
// Both operands are staged in LDS as [row][k] (contraction contiguous, padded pitch) so the MFMA
// fragments are single 16-byte LDS reads.  An operand whose memory layout is already contraction
// contiguous is copied with 16-byte accesses; one that is contiguous along its row index (the
// gathered feature rows of wgrad, A^T, B) is transposed on the way in with 2-byte LDS writes.
// X plays the MFMA "A" role so that a lane ends up with 4 consecutive n of one m: the epilogue
// writes 8-byte pieces that are contiguous in the row-major output.
#pragma once
#include "common.h"

namespace cummhip {

struct TileGemmParams {
  const void *X;  // operand indexed by n
  const void *Y;  // operand indexed by m
  void *C;
  const void *D;  // source; ldd == 0 -> bias over n
  int64_t ldx, ldy;        // K_CONTIG: stride between rows; else stride between k slices
  int64_t ldc, ldd;        // stride between output rows m
  int64_t c_off;           // element offset added per blockIdx.y / n_tiles_per_r (wgrad: r * C)
  const int32_t *x_gather; // non-K_CONTIG only: k -> memory row (wgrad: indices, by o or by pos)
  const int32_t *y_gather; // non-K_CONTIG only: k -> memory row (wgrad: mask_argsort)
  const uint32_t *red_mask;  // wgrad: per mask_width positions, NULL otherwise
  int32_t num_red_mask, mask_width;
  uint32_t mask_filter;
  int32_t m, n, k;         // wgrad: m = K, n = C (per offset), k = positions
  int32_t n_idx;           // row length of the [kv, n_idx] x_gather table
  int32_t rows_x, rows_y;  // gathered row numbers outside [0, rows) count as absent
  int32_t kv;              // kernel offsets (1 for plain GEMM)
  int32_t x_gather_via_y;  // wgrad: x row = x_gather[r * n_idx + y_gather[k]]
  float alpha, beta, act_alpha;
  int32_t act;
  int32_t split_k;
  int32_t *sem;            // [grid.x * grid.y] zeroed before launch (serial split-K)
  int32_t spin_limit;      // bound on semaphore polls
  int32_t *timeouts;       // counts the slices whose wait ran into the bound (the host reports them)
  // plain GEMM: slice z owns the contiguous range of k-steps [z * per, (z + 1) * per), per =
  // ceil(steps / split_k) (GemmUtils::get_gemm_k_size_per_split, include/tensorview/gemm/core/utils.h:30-37
  // of the reference); backward-weight: slices interleave (z, z + split_k, ...)
  int32_t split_contig;
};

// XK / YK: operand is contraction-contiguous in memory.  BM x BN 16x16 blocks per wave, 2x2 waves.
// WIDE: four-byte outputs (s32 for s8 operands, f32 for f16 / bf16 operands): the accumulators
// through a linear combination in the output type, integer arithmetic for s32 ("s8,s8,s32,s32,s32",
// cumm/gemm/main.py:350-364 of the reference; LinearCombination with dcomp = s32,
// cumm/gemm/output_op/linear.py:54-146).
template <class T, bool XK, bool YK, int BM, int BN, int KSTEPS, bool WIDE = false>
__global__ __launch_bounds__(256) void tilegemm_kernel(const TileGemmParams p) {
  using E = Elem<T>;
  using AccV = typename E::AccV;
  constexpr int TM = 2 * BM * 16;
  constexpr int TN = 2 * BN * 16;
  constexpr int TK = KSTEPS * E::kMfmaK;       // contraction elements per step
  constexpr int PV = E::kPerVec;               // elements per 16 bytes
  constexpr int PITCH = TK + PV;               // elements; keeps rows 16-byte aligned
  constexpr int KP = TK / PV;                  // 16-byte pieces per row
  __shared__ __attribute__((aligned(16))) char lds_raw[(TM + TN) * PITCH * E::kBytes];
  char *lds_x = lds_raw;
  char *lds_y = lds_raw + TN * PITCH * E::kBytes;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int l16 = lane & 15, q = lane >> 4;

  const int n_tiles = (p.n + TN - 1) / TN;   // per kernel offset
  const int r_off = blockIdx.y / n_tiles;    // kernel offset (0 for plain GEMM)
  const int n0 = (blockIdx.y % n_tiles) * TN;
  const int m0 = blockIdx.x * TM;
  const int z = blockIdx.z;
  if (p.kv > 1 && !((p.mask_filter >> r_off) & 1u)) return;

  AccV acc[BM][BN];
#pragma unroll
  for (int i = 0; i < BM; ++i)
#pragma unroll
    for (int j = 0; j < BN; ++j) acc[i][j] = AccV{0, 0, 0, 0};

  const int steps = (p.k + TK - 1) / TK;
  const int rate = p.red_mask ? p.mask_width / TK : 1;

  auto step_live = [&](int s) -> bool {
    if (p.red_mask == nullptr) return true;
    const int mi = s / rate;
    const uint32_t mw = mi < p.num_red_mask ? p.red_mask[mi] : 0u;
    return (mw >> r_off) & 1u;
  };
  const int per_slice = (steps + p.split_k - 1) / p.split_k;
  const int s_begin = p.split_contig ? z * per_slice : z;
  const int s_end = p.split_contig ? (steps < (z + 1) * per_slice ? steps : (z + 1) * per_slice) : steps;
  const int s_inc = p.split_contig ? 1 : p.split_k;
  auto next_live = [&](int s) -> int {
    while (s < s_end && !step_live(s)) s += s_inc;
    return s < s_end ? s : -1;
  };

  // ---- per-thread staging assignment
  // K-contiguous operand: granule = (row, piece): rows x KP pieces of 16 bytes.
  // Row-contiguous operand: granule = (k, piece of PV rows): TK x rows/PV.
  constexpr int XG = XK ? TN * KP : TK * (TN / PV);
  constexpr int YG = YK ? TM * KP : TK * (TM / PV);
  constexpr int XPT = (XG + 255) / 256, YPT = (YG + 255) / 256;
  v4i xreg[XPT], yreg[YPT];

  const char *xb = reinterpret_cast<const char *>(p.X);
  const char *yb = reinterpret_cast<const char *>(p.Y);

  auto gather_row = [&](bool is_x, int kk) -> int {
    // memory row holding contraction index kk of a row-contiguous operand
    if (kk >= p.k) return -1;
    int row = kk;
    if (is_x) {
      if (p.x_gather_via_y) {
        int o = p.y_gather ? p.y_gather[kk] : kk;
        row = (o >= 0 && o < p.n_idx) ? p.x_gather[(int64_t)r_off * p.n_idx + o] : -1;
      } else if (p.x_gather) {
        row = p.x_gather[kk];
      }
      if (row >= p.rows_x) row = -1;
    } else {
      if (p.y_gather) row = p.y_gather[kk];
      if (row >= p.rows_y) row = -1;
    }
    return row;
  };

  auto load_tiles = [&](int s) {
    const int k0 = s * TK;
    if constexpr (XK) {
#pragma unroll
      for (int i = 0; i < XPT; ++i) {
        const int id = tid + i * 256;
        v4i v = {0, 0, 0, 0};
        if (id < XG) {
          const int row = n0 + id / KP, kk = k0 + (id % KP) * PV;
          if (row < p.n && kk < p.k)
            v = *reinterpret_cast<const v4i *>(xb + ((int64_t)row * p.ldx + kk) * E::kBytes);
        }
        xreg[i] = v;
      }
    } else {
#pragma unroll
      for (int i = 0; i < XPT; ++i) {
        const int id = tid + i * 256;
        v4i v = {0, 0, 0, 0};
        if (id < XG) {
          const int kl = id % TK, piece = id / TK;  // k fastest: conflict-free transposed writes
          const int col = n0 + piece * PV;
          const int row = gather_row(true, k0 + kl);
          if (row >= 0 && col < p.n)
            v = *reinterpret_cast<const v4i *>(xb + ((int64_t)row * p.ldx + col) * E::kBytes);
        }
        xreg[i] = v;
      }
    }
    if constexpr (YK) {
#pragma unroll
      for (int i = 0; i < YPT; ++i) {
        const int id = tid + i * 256;
        v4i v = {0, 0, 0, 0};
        if (id < YG) {
          const int row = m0 + id / KP, kk = k0 + (id % KP) * PV;
          if (row < p.m && kk < p.k)
            v = *reinterpret_cast<const v4i *>(yb + ((int64_t)row * p.ldy + kk) * E::kBytes);
        }
        yreg[i] = v;
      }
    } else {
#pragma unroll
      for (int i = 0; i < YPT; ++i) {
        const int id = tid + i * 256;
        v4i v = {0, 0, 0, 0};
        if (id < YG) {
          const int kl = id % TK, piece = id / TK;
          const int col = m0 + piece * PV;
          const int row = gather_row(false, k0 + kl);
          if (row >= 0 && col < p.m)
            v = *reinterpret_cast<const v4i *>(yb + ((int64_t)row * p.ldy + col) * E::kBytes);
        }
        yreg[i] = v;
      }
    }
  };

  auto store_tiles = [&]() {
    if constexpr (XK) {
#pragma unroll
      for (int i = 0; i < XPT; ++i) {
        const int id = tid + i * 256;
        if (id < XG)
          *reinterpret_cast<v4i *>(lds_x + ((id / KP) * PITCH + (id % KP) * PV) * E::kBytes) = xreg[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < XPT; ++i) {
        const int id = tid + i * 256;
        if (id < XG) {
          const int kl = id % TK, piece = id / TK;
          if constexpr (E::kBytes == 2) {
            const uint16_t *src = reinterpret_cast<const uint16_t *>(&xreg[i]);
            uint16_t *dst = reinterpret_cast<uint16_t *>(lds_x);
#pragma unroll
            for (int e = 0; e < PV; ++e) dst[(piece * PV + e) * PITCH + kl] = src[e];
          } else {
            const uint8_t *src = reinterpret_cast<const uint8_t *>(&xreg[i]);
            uint8_t *dst = reinterpret_cast<uint8_t *>(lds_x);
#pragma unroll
            for (int e = 0; e < PV; ++e) dst[(piece * PV + e) * PITCH + kl] = src[e];
          }
        }
      }
    }
    if constexpr (YK) {
#pragma unroll
      for (int i = 0; i < YPT; ++i) {
        const int id = tid + i * 256;
        if (id < YG)
          *reinterpret_cast<v4i *>(lds_y + ((id / KP) * PITCH + (id % KP) * PV) * E::kBytes) = yreg[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < YPT; ++i) {
        const int id = tid + i * 256;
        if (id < YG) {
          const int kl = id % TK, piece = id / TK;
          if constexpr (E::kBytes == 2) {
            const uint16_t *src = reinterpret_cast<const uint16_t *>(&yreg[i]);
            uint16_t *dst = reinterpret_cast<uint16_t *>(lds_y);
#pragma unroll
            for (int e = 0; e < PV; ++e) dst[(piece * PV + e) * PITCH + kl] = src[e];
          } else {
            const uint8_t *src = reinterpret_cast<const uint8_t *>(&yreg[i]);
            uint8_t *dst = reinterpret_cast<uint8_t *>(lds_y);
#pragma unroll
            for (int e = 0; e < PV; ++e) dst[(piece * PV + e) * PITCH + kl] = src[e];
          }
        }
      }
    }
  };

  // ---- main loop: steps z, z + split, ... (slices interleave, cumm/gemm/blockmma/mma.py:634-655
  // of the reference); steps whose reduced mask lacks this offset's bit are skipped.
  int s = next_live(s_begin);
  if (s >= 0) load_tiles(s);
  while (s >= 0) {
    store_tiles();
    __syncthreads();
    const int s_next = next_live(s + s_inc);
    if (s_next >= 0) load_tiles(s_next);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      v4i xf[BN], yf[BM];
#pragma unroll
      for (int j = 0; j < BN; ++j)
        xf[j] = *reinterpret_cast<const v4i *>(
            lds_x + (((wn * BN + j) * 16 + l16) * PITCH + ks * E::kMfmaK + q * PV) * E::kBytes);
#pragma unroll
      for (int i = 0; i < BM; ++i)
        yf[i] = *reinterpret_cast<const v4i *>(
            lds_y + (((wm * BM + i) * 16 + l16) * PITCH + ks * E::kMfmaK + q * PV) * E::kBytes);
#pragma unroll
      for (int i = 0; i < BM; ++i)
#pragma unroll
        for (int j = 0; j < BN; ++j) acc[i][j] = E::mfma(xf[j], yf[i], acc[i][j]);
    }
    __syncthreads();
    s = s_next;
  }

  // ---- serial split-K: slice z waits until the slices before it have written
  // (tv::Semaphore, include/tensorview/gemm/arch/semaphore.h:37-100; use in
  //  cumm/conv/kernel.py:960-968,1004-1014,1068-1083 of the reference)
  int32_t *lock = nullptr;
  float beta = p.beta;
  if (p.split_k > 1) {
    lock = p.sem + (blockIdx.x + blockIdx.y * gridDim.x);
    if (tid == 0) {
      int spins = 0;
      bool mine = __hip_atomic_load(lock, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) == z;
      while (!mine && spins < p.spin_limit) {
        __builtin_amdgcn_s_sleep(8);
        ++spins;
        mine = __hip_atomic_load(lock, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) == z;
      }
      // The wait is bounded so that no wave can spin for ever.  A slice that gives up goes on
      // without its turn - the sum it writes is then not to be trusted - and says so: the host
      // reports the count as an error at its next synchronisation.
      if (!mine && p.timeouts != nullptr)
        __hip_atomic_fetch_add(p.timeouts, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (z > 0) beta = 1.0f;
  }
  const bool read_src = beta != 0.0f;

  // lane (l16, q) holds, for block (i, j): m = m0 + (wm*BM+i)*16 + l16, n = n0 + (wn*BN+j)*16 + 4q + r
#pragma unroll
  for (int i = 0; i < BM; ++i) {
    const int mm = m0 + (wm * BM + i) * 16 + l16;
    if (mm >= p.m) continue;
#pragma unroll
    for (int j = 0; j < BN; ++j) {
      const int nn = n0 + (wn * BN + j) * 16 + 4 * q;
      if (nn >= p.n) continue;
      const int64_t coff = (int64_t)mm * p.ldc + (int64_t)r_off * p.c_off + nn;
      const int64_t doff = (int64_t)mm * p.ldd + (p.ldd ? (int64_t)r_off * p.c_off : 0) + nn;
      if constexpr (WIDE) {
        int32_t *cp = reinterpret_cast<int32_t *>(p.C) + coff;
        v4i sv = {0, 0, 0, 0};
        if (read_src) sv = *reinterpret_cast<const v4i *>((z > 0) ? cp : reinterpret_cast<const int32_t *>(p.D) + doff);
        v4i ov;
        if constexpr (E::kBytes == 1) {
          const uint32_t ai = (uint32_t)(int)p.alpha, bi = (uint32_t)(int)beta, la = (uint32_t)(int)p.act_alpha;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            int t = (int)(ai * (uint32_t)acc[i][j][r] + (read_src ? bi * (uint32_t)sv[r] : 0u));
            if (p.act == 1) t = t > 0 ? t : 0;
            else if (p.act == 3) t = t >= 0 ? t : (int)((uint32_t)t * la);
            ov[r] = t;
          }
        } else {
          const v4f sf = __builtin_bit_cast(v4f, sv);
          v4f of;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float t = read_src ? __builtin_fmaf(p.alpha, acc[i][j][r], beta * sf[r]) : p.alpha * acc[i][j][r];
            of[r] = apply_act(t, p.act, p.act_alpha);
          }
          ov = __builtin_bit_cast(v4i, of);
        }
        *reinterpret_cast<v4i *>(cp) = ov;
      } else if constexpr (E::kBytes == 2) {
        uint16_t *cp = reinterpret_cast<uint16_t *>(p.C) + coff;
        uint2 sv = {0, 0};
        if (read_src) {
          const uint16_t *dp = (z > 0) ? cp : reinterpret_cast<const uint16_t *>(p.D) + doff;
          sv = *reinterpret_cast<const uint2 *>(dp);
        }
        const uint16_t *sh = reinterpret_cast<const uint16_t *>(&sv);
        uint2 ov;
        uint16_t *oh = reinterpret_cast<uint16_t *>(&ov);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float t = read_src ? __builtin_fmaf(p.alpha, acc[i][j][r], beta * E::to_float(sh[r]))
                             : p.alpha * acc[i][j][r];
          t = apply_act(t, p.act, p.act_alpha);
          oh[r] = E::from_float(t);
        }
        *reinterpret_cast<uint2 *>(cp) = ov;
      } else {
        int8_t *cp = reinterpret_cast<int8_t *>(p.C) + coff;
        uint32_t sv = 0;
        if (read_src) {
          const int8_t *dp = (z > 0) ? cp : reinterpret_cast<const int8_t *>(p.D) + doff;
          sv = *reinterpret_cast<const uint32_t *>(dp);
        }
        const int8_t *sb = reinterpret_cast<const int8_t *>(&sv);
        uint32_t ov;
        int8_t *ob = reinterpret_cast<int8_t *>(&ov);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float t = read_src ? __builtin_fmaf(p.alpha, (float)acc[i][j][r], beta * (float)sb[r])
                             : p.alpha * (float)acc[i][j][r];
          t = apply_act(t, p.act, p.act_alpha);
          ob[r] = (int8_t)f32_to_s8(t);
        }
        *reinterpret_cast<uint32_t *>(cp) = ov;
      }
    }
  }

  if (p.split_k > 1) {
    __threadfence();
    __syncthreads();
    if (tid == 0) {
      const int nxt = (z + 1 == p.split_k) ? 0 : z + 1;
      __hip_atomic_store(lock, nxt, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace cummhip
