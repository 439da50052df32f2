// Gather-rows x small-weight GEMM with a scatter epilogue for gfx950.
//
// One kernel family covers the mask-based sparse-convolution forward and
// backward-input passes and the ShuffleAC (gather A rows / scatter C rows) GEMM:
//
//   for each output position pos (row o = out_rows[pos]):
//     acc[o, :] = sum over kernel offsets k in the tile mask of  A[gather(k, o), :] @ W_k
//     C[o, :]   = epilogue(acc[o, :], D[o, :])
//
// Mapping to the hardware (wave64, 16x16 MFMA):
//   * the product is computed transposed, D^T = W_k^T * A^T, so that the gathered rows are the
//     MFMA "B" operand and every lane ends up holding TN/4 *contiguous* output channels of ONE
//     output row: the epilogue reads the source row and writes the result row with 16-byte
//     accesses and no LDS transpose, and no two lanes of different workgroups touch one row
//     (atomic-free scatter);
//   * a lane (m = lane%16, q = lane/16) needs, for row m, 16*KS contiguous bytes of the gathered
//     row per channel chunk: they are loaded from global memory straight into the MFMA operand
//     registers (the order of the contraction index inside a chunk is permuted identically for
//     both operands, which leaves the product unchanged), so gathered rows never pass through LDS;
//   * the weight slice of the current (offset, channel chunk) is staged by the whole workgroup
//     into LDS in fragment order (double buffered, one barrier per step) and read back with
//     conflict-free 16-byte reads;
//   * each wave owns RB blocks of 16 rows; a block none of whose rows has a pair at offset k is
//     skipped (its contribution would be exactly zero).
#pragma once
#include "common.h"

namespace cummhip {

struct RowGemmParams {
  const void *A;   // gathered operand, rows of lda elements
  const void *W;   // weights
  void *C;         // output rows of ldc elements
  const void *D;   // source rows of ldd elements (ldd == 0: one row shared by all = bias)
  const int32_t *out_rows;  // [n_pos] position -> output row, NULL = identity
  const int32_t *gather;    // conv: [kv, n_idx] indexed by output row; gemm: [n_pos] or NULL
  const uint32_t *mask;     // [n_pos] per-position offset mask, NULL = single offset
  uint32_t *mask_out;       // [tiles] or NULL
  const float *scale;       // int8 epilogue
  const float *bias;
  int64_t lda, ldc, ldd;
  int64_t w_stride_n, w_stride_k, w_stride_c;  // element strides: out channel, offset, contraction
  int32_t n_pos, n_idx, rows_a, rows_c;
  int32_t c_in, k_out, kv;
  uint32_t mask_filter;
  int32_t reverse_mask, exit_on_empty, gather_by_pos;
  float alpha, beta, act_alpha, act_beta;
  int32_t act;
  int32_t int8_epilogue;  // scale/bias requantisation instead of alpha/beta
  int32_t read_source;    // D is read (beta != 0)
  int32_t xcd_swizzle;    // remap blockIdx.x so that neighbouring tiles share an XCD
};

// T: element tag; NW: waves per workgroup; RB: 16-row blocks per wave; TN: output channels per
// workgroup; KS: 16-byte fragments per lane per channel chunk; WT: weight is contiguous along the
// output channel (needs a transposing stage) instead of along the contraction.
template <class T, int NW, int RB, int TN, int KS, bool WT>
__global__ __launch_bounds__(NW * 64) void rowgemm_kernel(const RowGemmParams p) {
  using E = Elem<T>;
  using AccV = typename E::AccV;
  constexpr int TM = NW * RB * 16;
  constexpr int NB = TN / 16;               // MFMA row blocks (output channel blocks)
  constexpr int CPL = TN / 4;               // output channels per lane
  constexpr int CHUNK_E = 4 * KS * E::kPerVec;  // contraction elements per chunk
  constexpr int STAGE_V = NB * KS * 64;     // 16-byte vectors per LDS stage
  constexpr int NT = NW * 64;

  __shared__ v4i lds_w[2][STAGE_V];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 15;
  const int q = lane >> 4;

  int tile = blockIdx.x;
  if (p.xcd_swizzle) {
    // workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous range of tiles
    const int nt = gridDim.x;
    const int per = nt >> 3;
    if (tile < per * 8) tile = (tile & 7) * per + (tile >> 3);
  }
  const int n0 = blockIdx.y * TN;
  const int pos_base = tile * TM;

  // ---- tile mask: OR over the tile's positions (cumm/conv/kernel.py:844-889 of the reference)
  uint32_t kmask;
  if (p.mask != nullptr) {
    uint32_t mk = 0;
#pragma unroll
    for (int i = 0; i < (TM + 63) / 64; ++i) {
      const int pp = pos_base + i * 64 + lane;
      if (i * 64 + lane < TM && pp < p.n_pos) mk |= p.mask[pp];
    }
    kmask = wave_or(mk) & p.mask_filter;
    kmask = __builtin_amdgcn_readfirstlane(kmask);
    if (p.mask_out != nullptr && tid == 0 && blockIdx.y == 0) p.mask_out[tile] = kmask;
    if (p.exit_on_empty && kmask == 0) return;
    if (p.reverse_mask) kmask = __builtin_bitreverse32(kmask) >> (32 - p.kv);
    if (p.kv < 32) kmask &= (1u << p.kv) - 1u;
  } else {
    kmask = 1u;
  }

  // ---- rows owned by this lane
  int out_row[RB];
  int key[RB];  // what the gather table is indexed with
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int pos = pos_base + (wave * RB + rb) * 16 + m;
    int o = -1;
    if (pos < p.n_pos) o = p.out_rows ? p.out_rows[pos] : pos;
    out_row[rb] = o;
    key[rb] = p.gather_by_pos ? (pos < p.n_pos ? pos : -1) : o;
  }

  AccV acc[RB][NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[rb][nb] = AccV{0, 0, 0, 0};

  const int n_chunks = (p.c_in + CHUNK_E - 1) / CHUNK_E;
  const char *a_base = reinterpret_cast<const char *>(p.A);
  const int64_t a_row_bytes = p.lda * E::kBytes;

  auto load_idx = [&](int k, int (&idx)[RB]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      int v = -1;
      const int kk = key[rb];
      if (kk >= 0) {
        if (p.gather != nullptr) {
          if (p.gather_by_pos || kk < p.n_idx) v = p.gather[(int64_t)k * p.n_idx + kk];
        } else {
          v = kk;
        }
      }
      if (v >= p.rows_a) v = -1;
      idx[rb] = v;
    }
  };

  auto load_a = [&](const int (&idx)[RB], int chunk, v4i (&frag)[RB][KS]) {
    const int e0 = chunk * CHUNK_E + q * KS * E::kPerVec;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const char *row = a_base + (int64_t)(idx[rb] < 0 ? 0 : idx[rb]) * a_row_bytes;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int e = e0 + s * E::kPerVec;
        v4i v = {0, 0, 0, 0};
        if (idx[rb] >= 0 && e < p.c_in) v = *reinterpret_cast<const v4i *>(row + (int64_t)e * E::kBytes);
        frag[rb][s] = v;
      }
    }
  };

  // weight staging: granule id -> (output channel, 16-byte piece of the chunk)
  constexpr int GRAN = TN * 4 * KS;  // 16-byte granules per stage
  constexpr int GPT = (GRAN + NT - 1) / NT;
  const char *w_base = reinterpret_cast<const char *>(p.W);

  auto lds_slot = [&](int n_local, int g) -> int {
    // lane (m', q') of the reading wave holds channel n0 + q'*CPL + nb*4 + r as MFMA row 4*q'+r
    const int qo = n_local / CPL;
    const int rem = n_local % CPL;
    const int nb = rem >> 2;
    const int r = rem & 3;
    const int rho = qo * 4 + r;
    const int qq = g / KS;
    const int s = g % KS;
    return (nb * KS + s) * 64 + qq * 16 + rho;
  };

  v4i wreg[GPT];
  auto load_w = [&](int k, int chunk) {
    if constexpr (!WT) {
#pragma unroll
      for (int i = 0; i < GPT; ++i) {
        const int id = tid + i * NT;
        v4i v = {0, 0, 0, 0};
        if (id < GRAN) {
          const int n_local = id / (4 * KS);
          const int g = id % (4 * KS);
          const int n = n0 + n_local;
          const int e = chunk * CHUNK_E + g * E::kPerVec;
          if (n < p.k_out && e < p.c_in) {
            const int64_t off = (int64_t)n * p.w_stride_n + (int64_t)k * p.w_stride_k + e;
            v = *reinterpret_cast<const v4i *>(w_base + off * E::kBytes);
          }
        }
        wreg[i] = v;
      }
    } else {
      // granule = kPerVec consecutive OUTPUT channels at one contraction index
#pragma unroll
      for (int i = 0; i < GPT; ++i) {
        const int id = tid + i * NT;
        v4i v = {0, 0, 0, 0};
        if (id < GRAN) {
          constexpr int NG = TN / E::kPerVec;  // granules along the output channels
          const int c_local = id / NG;         // contraction index inside the chunk
          const int ng = id % NG;
          const int n = n0 + ng * E::kPerVec;
          const int e = chunk * CHUNK_E + c_local;
          if (n < p.k_out && e < p.c_in) {
            const int64_t off = (int64_t)e * p.w_stride_c + (int64_t)k * p.w_stride_k + n;
            v = *reinterpret_cast<const v4i *>(w_base + off * E::kBytes);
          }
        }
        wreg[i] = v;
      }
    }
  };

  auto store_w = [&](int buf) {
    if constexpr (!WT) {
#pragma unroll
      for (int i = 0; i < GPT; ++i) {
        const int id = tid + i * NT;
        if (id < GRAN) lds_w[buf][lds_slot(id / (4 * KS), id % (4 * KS))] = wreg[i];
      }
    } else {
      constexpr int NG = TN / E::kPerVec;
#pragma unroll
      for (int i = 0; i < GPT; ++i) {
        const int id = tid + i * NT;
        if (id < GRAN) {
          const int c_local = id / NG;
          const int ng = id % NG;
          const int g = c_local / E::kPerVec;  // 16-byte piece along the contraction
          const int j = c_local % E::kPerVec;  // element inside the piece
          if constexpr (E::kBytes == 2) {
            uint16_t *dst = reinterpret_cast<uint16_t *>(&lds_w[buf][0]);
            const uint16_t *src = reinterpret_cast<const uint16_t *>(&wreg[i]);
#pragma unroll
            for (int x = 0; x < 8; ++x) dst[lds_slot(ng * 8 + x, g) * 8 + j] = src[x];
          } else {
            uint8_t *dst = reinterpret_cast<uint8_t *>(&lds_w[buf][0]);
            const uint8_t *src = reinterpret_cast<const uint8_t *>(&wreg[i]);
#pragma unroll
            for (int x = 0; x < 16; ++x) dst[lds_slot(ng * 16 + x, g) * 16 + j] = src[x];
          }
        }
      }
    }
  };

  if (kmask != 0) {
    // ---- software pipeline over (offset, chunk) steps
    uint32_t rem = kmask;
    int k_cur = __builtin_ctz(rem);
    rem &= rem - 1;
    int k_nxt = rem ? __builtin_ctz(rem) : -1;
    if (rem) rem &= rem - 1;

    int idx_cur[RB], idx_nxt[RB];
    load_idx(k_cur, idx_cur);
    if (k_nxt >= 0) load_idx(k_nxt, idx_nxt);

    v4i a_nxt[RB][KS];
    load_a(idx_cur, 0, a_nxt);
    load_w(k_cur, 0);
    bool any_nxt[RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) any_nxt[rb] = __ballot(idx_cur[rb] >= 0) != 0;

    int chunk = 0;
    int buf = 0;
    bool more = true;
    while (more) {
      v4i a_cur[RB][KS];
      bool any_cur[RB];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        any_cur[rb] = any_nxt[rb];
#pragma unroll
        for (int s = 0; s < KS; ++s) a_cur[rb][s] = a_nxt[rb][s];
      }
      store_w(buf);
      __syncthreads();

      // advance to the next step and start its loads
      if (chunk + 1 < n_chunks) {
        ++chunk;
      } else {
        chunk = 0;
        k_cur = k_nxt;
        if (k_cur >= 0) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) idx_cur[rb] = idx_nxt[rb];
          k_nxt = rem ? __builtin_ctz(rem) : -1;
          if (rem) rem &= rem - 1;
          if (k_nxt >= 0) load_idx(k_nxt, idx_nxt);
        }
      }
      more = k_cur >= 0;
      if (more) {
        load_a(idx_cur, chunk, a_nxt);
        load_w(k_cur, chunk);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) any_nxt[rb] = __ballot(idx_cur[rb] >= 0) != 0;
      }

      // ---- MFMA over the staged weight slice
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        v4i wf[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) wf[s] = lds_w[buf][(nb * KS + s) * 64 + lane];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          if (any_cur[rb]) {
#pragma unroll
            for (int s = 0; s < KS; ++s) acc[rb][nb] = E::mfma(wf[s], a_cur[rb][s], acc[rb][nb]);
          }
        }
      }
      buf ^= 1;
    }
  }

  // ---- epilogue: lane (m, q) owns channels [n0 + q*CPL, n0 + (q+1)*CPL) of row out_row[rb]
  const int ch0 = n0 + q * CPL;
  if constexpr (E::kBytes == 2) {
    constexpr int NG = CPL / 8;  // 16-byte groups of 8 channels
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int o = out_row[rb];
      if (o < 0 || o >= p.rows_c) continue;
      uint16_t *crow = reinterpret_cast<uint16_t *>(p.C) + (int64_t)o * p.ldc;
      const uint16_t *drow = reinterpret_cast<const uint16_t *>(p.D) + (int64_t)o * p.ldd;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int ch = ch0 + g * 8;
        if (ch >= p.k_out) continue;
        v4i src = {0, 0, 0, 0};
        if (p.read_source) src = *reinterpret_cast<const v4i *>(drow + ch);
        const uint16_t *sh = reinterpret_cast<const uint16_t *>(&src);
        v4i outv;
        uint16_t *oh = reinterpret_cast<uint16_t *>(&outv);
#pragma unroll
        for (int x = 0; x < 8; ++x) {
          const float a = acc[rb][g * 2 + (x >> 2)][x & 3];
          float t;
          if (p.read_source) {
            t = __builtin_fmaf(p.alpha, a, p.beta * E::to_float(sh[x]));
          } else {
            t = p.alpha * a;
          }
          t = apply_act(t, p.act, p.act_alpha);
          oh[x] = E::from_float(t);
        }
        *reinterpret_cast<v4i *>(crow + ch) = outv;
      }
    }
  } else {
    // s8 output rows: 16 channels per 16-byte store
    constexpr int NG = CPL / 16;
    static_assert(CPL % 16 == 0, "s8 kernels need TN >= 64");
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int o = out_row[rb];
      if (o < 0 || o >= p.rows_c) continue;
      int8_t *crow = reinterpret_cast<int8_t *>(p.C) + (int64_t)o * p.ldc;
      const int8_t *drow = reinterpret_cast<const int8_t *>(p.D) + (int64_t)o * p.ldd;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int ch = ch0 + g * 16;
        if (ch >= p.k_out) continue;
        v4i src = {0, 0, 0, 0};
        if (p.read_source) src = *reinterpret_cast<const v4i *>(drow + ch);
        const int8_t *sb = reinterpret_cast<const int8_t *>(&src);
        v4i outv;
        int8_t *ob = reinterpret_cast<int8_t *>(&outv);
#pragma unroll
        for (int x = 0; x < 16; ++x) {
          const int a = acc[rb][g * 4 + (x >> 2)][x & 3];
          float t;
          if (p.int8_epilogue) {
            // Int8Inference: scale*acc + bias, then beta*source + that
            // (cumm/gemm/output_op/linear.py:279-325 of the reference)
            t = __builtin_fmaf(p.scale[ch + x], (float)a, p.bias[ch + x]);
            if (p.read_source) t = __builtin_fmaf(p.beta, (float)sb[x], t);
          } else if (p.read_source) {
            t = __builtin_fmaf(p.alpha, (float)a, p.beta * (float)sb[x]);
          } else {
            t = p.alpha * (float)a;
          }
          t = apply_act(t, p.act, p.act_alpha);
          ob[x] = (int8_t)f32_to_s8(t);
        }
        *reinterpret_cast<v4i *>(crow + ch) = outv;
      }
    }
  }
}

}  // namespace cummhip
