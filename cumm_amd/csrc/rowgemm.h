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
//   * a lane (m = lane%16, q = lane/16) needs, for row m, KS 16-byte pieces of the gathered row per
//     channel chunk (piece s*4 + q for fragment s): they are loaded from global memory straight into the MFMA operand
//     registers (the order of the contraction index inside a chunk is permuted identically for
//     both operands, which leaves the product unchanged), so gathered rows never pass through LDS;
//   * all gathers go through buffer descriptors: an absent pair (index -1), a row past the end or
//     a channel past C is an out-of-range offset that the hardware answers with zeros, so the hot
//     loop has no divergent branches;
//   * kernel offsets are processed in batches of B: the gathered rows of a whole batch are
//     requested together and the pair-table entries and weight slices of the NEXT batch are
//     requested before the MFMAs of the current one, so a batch costs one memory round trip;
//     weight slices are staged by the whole workgroup into LDS in fragment order (double
//     buffered) and read back with conflict-free 16-byte reads;
//   * tiles are handed out heaviest first; each wave owns RB blocks of 16 rows and skips a block
//     none of whose rows has a pair at offset k (its contribution would be exactly zero).
#pragma once
#include <type_traits>

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
  uint32_t a_bytes, w_bytes, c_bytes, d_bytes, gather_bytes;  // extents for the range checks
  int32_t n_pos, n_idx, rows_a, rows_c;
  int32_t c_in, k_out, kv;
  uint32_t mask_filter;
  int32_t reverse_mask, exit_on_empty, gather_by_pos;
  float alpha, beta, act_alpha, act_beta;
  int32_t act;
  int32_t int8_epilogue;  // scale/bias requantisation instead of alpha/beta
  int32_t read_source;    // D is read (beta != 0)
  // LDS-streaming kernel only: the contraction is walked in 2^chunk_shift chunks of one stage
  // row each (a step = one kernel offset x one chunk); 0 = the whole contraction fits a row
  int32_t chunk_shift;
  // LDS-streaming kernel, one column block: the first pair_tiles runs of 128 sorted positions are
  // taken as 128-row tiles (rowgemm_lds_mixed_kernel); 0 = 64-row tiles throughout
  int32_t pair_tiles;
  // ... or, when pair_tiles is 0 and this is not NULL, what the hint slot says: eight words
  // {mask pointer (two words), n_pos, mask_filter, light prefix in positions, ...} that input
  // preparation left for this mask array (light_hint_slot in launch.h); a slot that names another
  // array, length or filter says nothing
  const int32_t *hint_slot;
  // 32-bit mask words per position (1; 2 to 4 for kernel volumes above 32: see rowgemm_lds_tile)
  int32_t mask_words;
  // words the caller's mask_out array holds (a tile number beyond it is not written)
  int32_t n_mask_out;
  // non-zero: a row takes part in every kernel offset of its tile's mask (the reference's rule:
  // rows are gated by their pair-table entry alone, cumm/conv/sparse_iters.py:629-631), instead of
  // only in the offsets whose bit its own mask word has
  int32_t ungated_rows;
  // non-zero: the output rows are stored with the non-temporal hint (see kStreamStore)
  int32_t stream_stores;
  // non-zero (descriptors with num_stage 3): a contraction of more than 128 bytes is walked in
  // 64-byte chunks through three stages where the tile has such a kernel (128 x 128)
  int32_t small_stages;
};

// An offset no buffer contains: every operand is smaller than 2 GiB (checked on the host), and
// adding a scalar offset below 2 GiB to it cannot wrap back into range.
constexpr uint32_t kOob = 0x80000000u;

// Cache policy of the output stores when RowGemmParams::stream_stores is set: non-temporal.  A
// launch writes every output row once and never reads it back, and what the L2s still hold dirty
// when the last workgroup leaves is written back before the launch counts as finished; streamed
// stores are on their way to memory while the launch still runs (headline forward, 15 MB of
// output: 13.2 -> 12.4 us; write-through with sc1 instead: 13.2 us on a box where the plain stores
// gave 13.8).  The tail is at most the 32 MB the L2s hold, so larger launches gain little and
// lose the L2's merging of a row's pieces (84 MB of one-byte rows: 57.0 -> 59.2 us; 256 MB: 2 - 3 %
// slower): the host sets the flag for outputs up to kStreamStoreMaxBytes.  The same hint on the
// gathered row loads made the headline launch slower (16.4 us), and on the stores of the
// gather-GEMM-scatter kernel that keeps its weights in registers too (13.4 -> 14.5 us).
constexpr int kStreamStore = 2;   // aux bit 1 = nt
constexpr uint32_t kStreamStoreMaxBytes = 32u << 20;
template <class V>
__device__ __forceinline__ void store_out_b128(V v, __amdgpu_buffer_rsrc_t rs, uint32_t off, bool stream) {
  if (stream) __builtin_amdgcn_raw_buffer_store_b128(v, rs, off, 0, kStreamStore);
  else __builtin_amdgcn_raw_buffer_store_b128(v, rs, off, 0, 0);
}
template <class V>
__device__ __forceinline__ void store_out_b64(V v, __amdgpu_buffer_rsrc_t rs, uint32_t off, bool stream) {
  if (stream) __builtin_amdgcn_raw_buffer_store_b64(v, rs, off, 0, kStreamStore);
  else __builtin_amdgcn_raw_buffer_store_b64(v, rs, off, 0, 0);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}

// Four-byte outputs (s32 for s8 operands, f32 for f16 / bf16 operands; "s8,s8,s32,s32,s32" in
// cumm/gemm/main.py:350-364,500-523 of the reference): the accumulators themselves go through
// the linear combination, whose arithmetic type (dcomp) is then the output type: for s32 alpha
// and beta are converted to integers and alpha*acc + beta*src is integer arithmetic
// (LinearCombination, cumm/gemm/output_op/linear.py:54-146; UnaryActivation on integers,
// cumm/gemm/gemmmath/__init__.py:181-214).  One piece = four consecutive channels of one row.
template <class AccV>
__device__ __forceinline__ void store_wide_piece(const AccV &a, const RowGemmParams &p, __amdgpu_buffer_rsrc_t rs_c,
                                                 __amdgpu_buffer_rsrc_t rs_d, bool ok, int o, int ch) {
  const uint32_t coff = ok ? (uint32_t)((int64_t)o * p.ldc + ch) * 4u : kOob;
  v4i src = {0, 0, 0, 0};
  if (p.read_source) {
    const uint32_t doff = ok ? (uint32_t)((int64_t)o * p.ldd + ch) * 4u : kOob;
    src = __builtin_amdgcn_raw_buffer_load_b128(rs_d, doff, 0, 0);
  }
  v4i outv;
  if constexpr (std::is_same<AccV, v4i>::value) {
    // (unsigned arithmetic: wraps like the reference's int32 arithmetic, without undefined overflow)
    const uint32_t ai = (uint32_t)(int)p.alpha, bi = (uint32_t)(int)p.beta, la = (uint32_t)(int)p.act_alpha;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      int t = (int)(ai * (uint32_t)a[x] + (p.read_source ? bi * (uint32_t)src[x] : 0u));
      if (p.act == 1) t = t > 0 ? t : 0;
      else if (p.act == 3) t = t >= 0 ? t : (int)((uint32_t)t * la);
      outv[x] = t;
    }
  } else {
    const v4f sf = __builtin_bit_cast(v4f, src);
    v4f of;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const float t = p.read_source ? __builtin_fmaf(p.alpha, a[x], p.beta * sf[x]) : p.alpha * a[x];
      of[x] = apply_act(t, p.act, p.act_alpha);
    }
    outv = __builtin_bit_cast(v4i, of);
  }
  store_out_b128(outv, rs_c, coff, p.stream_stores != 0);
}

// T: element tag; NW: waves per workgroup; RB: 16-row blocks per wave; TN: output channels per
// workgroup; KS: 16-byte fragments per lane per channel chunk; WT: weight is contiguous along the
// output channel (needs a transposing stage) instead of along the contraction; B: kernel offsets
// per batch; WIDE: four-byte outputs (see store_wide_piece).
template <class T, int NW, int RB, int TN, int KS, bool WT, int B, bool WIDE = false>
__global__ __launch_bounds__(NW * 64) void rowgemm_kernel(const RowGemmParams p) {
  using E = Elem<T>;
  using AccV = typename E::AccV;
  constexpr int TM = NW * RB * 16;
  constexpr int NB = TN / 16;               // MFMA row blocks (output channel blocks)
  constexpr int CPL = TN / 4;               // output channels per lane
  constexpr int PV = E::kPerVec;
  constexpr int CHUNK_E = 4 * KS * PV;      // contraction elements per chunk
  constexpr int SLICE_V = NB * KS * 64;     // 16-byte vectors of one staged weight slice
  constexpr int NT = NW * 64;

  __shared__ v4i lds_w[2][B * SLICE_V];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 15;
  const int q = lane >> 4;

  // Tiles are handed out last-to-first: positions are sorted by ascending mask value, so the
  // tiles with the most kernel offsets (the longest running ones) sit at the end of the sorted
  // order and should start first, not last.
  const int tile = (int)gridDim.x - 1 - (int)blockIdx.x;
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
    if (p.mask_out != nullptr && tid == 0 && blockIdx.y == 0 && tile < p.n_mask_out) p.mask_out[tile] = kmask;
    if (p.exit_on_empty && kmask == 0) return;
    if (p.reverse_mask) kmask = __builtin_bitreverse32(kmask) >> (32 - p.kv);
    if (p.kv < 32) kmask &= (1u << p.kv) - 1u;
  } else {
    kmask = 1u;
  }

  // ---- rows owned by this lane
  int out_row[RB];
  uint32_t key_off[RB];  // byte offset of the lane's entry inside one row of the gather table
  bool key_ok[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int pos = pos_base + (wave * RB + rb) * 16 + m;
    int o = -1;
    if (pos < p.n_pos) o = p.out_rows ? p.out_rows[pos] : pos;
    out_row[rb] = o;
    const int key = p.gather_by_pos ? (pos < p.n_pos ? pos : -1) : o;
    key_ok[rb] = key >= 0 && key < p.n_idx;
    key_off[rb] = key_ok[rb] ? (uint32_t)key * 4u : kOob;
  }

  AccV acc[RB][NB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[rb][nb] = AccV{0, 0, 0, 0};

  const int n_chunks = (p.c_in + CHUNK_E - 1) / CHUNK_E;
  const uint32_t a_row_bytes = (uint32_t)p.lda * E::kBytes;
  const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(p.A, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(p.W, p.w_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(p.gather, p.gather ? p.gather_bytes : 0u);
  const bool has_gather = p.gather != nullptr;

  // pair-table entries of offset k for the lane's rows (raw: fix_idx() maps absent ones to -1)
  auto load_idx = [&](int k, int (&idx)[RB]) {
    const uint32_t base = (uint32_t)k * (uint32_t)p.n_idx * 4u;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      if (has_gather) {
        idx[rb] = __builtin_amdgcn_raw_buffer_load_b32(rs_g, key_ok[rb] ? base + key_off[rb] : kOob, 0, 0);
      } else {
        idx[rb] = (int)(key_off[rb] >> 2);
      }
    }
  };
  auto fix_idx = [&](int (&idx)[RB]) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
      if (!key_ok[rb] || idx[rb] >= p.rows_a) idx[rb] = -1;
  };

  auto load_a = [&](const int (&idx)[RB], int chunk, v4i (&frag)[RB][KS]) {
    // fragment s of lane quarter q is 16-byte piece s*4 + q of the chunk, so that one load
    // instruction touches a single 64-byte segment of each gathered row
    const int e0 = chunk * CHUNK_E + q * PV;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const uint32_t row = (uint32_t)idx[rb] * a_row_bytes;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int e = e0 + s * 4 * PV;
        const uint32_t off = (idx[rb] >= 0 && e < p.c_in) ? row + (uint32_t)e * E::kBytes : kOob;
        frag[rb][s] = __builtin_amdgcn_raw_buffer_load_b128(rs_a, off, 0, 0);
      }
    }
  };

  // weight staging: granule id -> (output channel, 16-byte piece of the chunk)
  constexpr int GRAN = TN * 4 * KS;  // 16-byte granules per offset
  constexpr int GPT = (GRAN + NT - 1) / NT;

  auto lds_slot = [&](int n_local, int g) -> int {
    // lane (m', q') of the reading wave holds channel n0 + q'*CPL + nb*4 + r as MFMA row 4*q'+r
    const int qo = n_local / CPL;
    const int rem = n_local % CPL;
    const int nb = rem >> 2;
    const int r = rem & 3;
    const int rho = qo * 4 + r;
    const int qq = g % 4;
    const int s = g / 4;
    // the low bits are XOR-swizzled so that the staging writes of a wave spread over all banks
    return (nb * KS + s) * 64 + qq * 16 + (rho ^ (qq << 2) ^ (nb & 3));
  };

  auto load_w = [&](int k, int chunk, v4i (&wreg)[GPT]) {
#pragma unroll
    for (int i = 0; i < GPT; ++i) {
      const int id = tid + i * NT;
      uint32_t off = kOob;
      if constexpr (!WT) {
        const int n = n0 + id / (4 * KS);
        const int e = chunk * CHUNK_E + (id % (4 * KS)) * PV;
        if (id < GRAN && n < p.k_out && e < p.c_in)
          off = (uint32_t)((int64_t)n * p.w_stride_n + (int64_t)k * p.w_stride_k + e) * E::kBytes;
      } else {
        // granule = PV consecutive OUTPUT channels at one contraction index
        constexpr int NG = TN / PV;
        const int n = n0 + (id % NG) * PV;
        const int e = chunk * CHUNK_E + id / NG;
        if (id < GRAN && n < p.k_out && e < p.c_in)
          off = (uint32_t)((int64_t)e * p.w_stride_c + (int64_t)k * p.w_stride_k + n) * E::kBytes;
      }
      wreg[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, off, 0, 0);
    }
  };

  auto store_w = [&](v4i *stage, const v4i (&wreg)[GPT]) {
    if constexpr (!WT) {
#pragma unroll
      for (int i = 0; i < GPT; ++i) {
        const int id = tid + i * NT;
        if (id < GRAN) stage[lds_slot(id / (4 * KS), id % (4 * KS))] = wreg[i];
      }
    } else {
      constexpr int NG = TN / PV;
#pragma unroll
      for (int i = 0; i < GPT; ++i) {
        const int id = tid + i * NT;
        if (id < GRAN) {
          const int c_local = id / NG;
          const int ng = id % NG;
          const int g = c_local / PV;  // 16-byte piece along the contraction
          const int j = c_local % PV;  // element inside the piece
          if constexpr (E::kBytes == 2) {
            uint16_t *dst = reinterpret_cast<uint16_t *>(stage);
            const uint16_t *src = reinterpret_cast<const uint16_t *>(&wreg[i]);
#pragma unroll
            for (int x = 0; x < 8; ++x) dst[lds_slot(ng * 8 + x, g) * 8 + j] = src[x];
          } else {
            uint8_t *dst = reinterpret_cast<uint8_t *>(stage);
            const uint8_t *src = reinterpret_cast<const uint8_t *>(&wreg[i]);
#pragma unroll
            for (int x = 0; x < 16; ++x) dst[lds_slot(ng * 16 + x, g) * 16 + j] = src[x];
          }
        }
      }
    }
  };

  // ---- steps: (batch of up to B offsets) x (channel chunk); the next step's pair-table entries
  // and weight slices are in flight while the current step computes
  if (kmask != 0) {
    uint32_t rem = kmask;
    auto take = [&](int (&ko)[B]) {
#pragma unroll
      for (int j = 0; j < B; ++j) {
        ko[j] = rem ? __builtin_ctz(rem) : -1;
        if (rem) rem &= rem - 1;
      }
    };
    int koff[B];
    take(koff);
    int chunk = 0;
    int idx[B][RB];
    v4i wreg[B][GPT];
#pragma unroll
    for (int j = 0; j < B; ++j) {
      if (koff[j] >= 0) {
        load_w(koff[j], 0, wreg[j]);
        load_idx(koff[j], idx[j]);
      }
    }
    int buf = 0;
    bool more = true;
    while (more) {
      // park the weight slices of this step in LDS (their requests went out a step ago)
#pragma unroll
      for (int j = 0; j < B; ++j)
        if (koff[j] >= 0) store_w(&lds_w[buf][j * SLICE_V], wreg[j]);
      if (chunk == 0) {
#pragma unroll
        for (int j = 0; j < B; ++j) {
          if (koff[j] >= 0) {
            fix_idx(idx[j]);
          } else {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) idx[j][rb] = -1;
          }
        }
      }
      // request every gathered row of the step
      v4i afrag[B][RB][KS];
      bool any[B][RB];
      int kcur[B];
#pragma unroll
      for (int j = 0; j < B; ++j) {
        kcur[j] = koff[j];
        if (koff[j] >= 0) load_a(idx[j], chunk, afrag[j]);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) any[j][rb] = koff[j] >= 0 && __ballot(idx[j][rb] >= 0) != 0;
      }
      // advance and request the next step's weight slices and pair-table entries
      if (chunk + 1 < n_chunks) {
        ++chunk;
#pragma unroll
        for (int j = 0; j < B; ++j)
          if (koff[j] >= 0) load_w(koff[j], chunk, wreg[j]);
      } else if (rem != 0) {
        chunk = 0;
        take(koff);
#pragma unroll
        for (int j = 0; j < B; ++j) {
          if (koff[j] >= 0) {
            load_w(koff[j], 0, wreg[j]);
            load_idx(koff[j], idx[j]);
          }
        }
      } else {
        more = false;
      }
      __syncthreads();  // this stage is written; every wave has left the other one
#pragma unroll
      for (int j = 0; j < B; ++j) {
        if (kcur[j] < 0) continue;
        const v4i *stage = &lds_w[buf][j * SLICE_V];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          v4i wf[KS];
#pragma unroll
          for (int s = 0; s < KS; ++s) wf[s] = stage[(nb * KS + s) * 64 + (lane ^ ((q << 2) ^ (nb & 3)))];
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            if (any[j][rb]) {
#pragma unroll
              for (int s = 0; s < KS; ++s) acc[rb][nb] = E::mfma(wf[s], afrag[j][rb][s], acc[rb][nb]);
            }
          }
        }
      }
      buf ^= 1;
    }
  }

  // ---- epilogue: lane (m, q) owns channels [n0 + q*CPL, n0 + (q+1)*CPL) of row out_row[rb]
  const __amdgpu_buffer_rsrc_t rs_c = make_rsrc(p.C, p.c_bytes);
  const __amdgpu_buffer_rsrc_t rs_d = make_rsrc(p.D, p.read_source ? p.d_bytes : 0u);
  const int ch0 = n0 + q * CPL;
  if constexpr (WIDE) {
    // lane (m, q): channels ch0 + 4*nb .. +3 of block nb, one 16-byte piece each
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int o = out_row[rb];
      const bool row_ok = o >= 0 && o < p.rows_c;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int ch = ch0 + nb * 4;
        store_wide_piece(acc[rb][nb], p, rs_c, rs_d, row_ok && ch < p.k_out, o, ch);
      }
    }
    return;
  }
  if constexpr (E::kBytes == 2) {
    constexpr int NG = CPL / 8;  // 16-byte groups of 8 channels
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int o = out_row[rb];
      const bool row_ok = o >= 0 && o < p.rows_c;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int ch = ch0 + g * 8;
        const bool ok = row_ok && ch < p.k_out;
        const uint32_t coff = ok ? (uint32_t)((int64_t)o * p.ldc + ch) * 2u : kOob;
        v4i src = {0, 0, 0, 0};
        if (p.read_source) {
          const uint32_t doff = ok ? (uint32_t)((int64_t)o * p.ldd + ch) * 2u : kOob;
          src = __builtin_amdgcn_raw_buffer_load_b128(rs_d, doff, 0, 0);
        }
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
        __builtin_amdgcn_raw_buffer_store_b128(outv, rs_c, coff, 0, 0);
      }
    }
  } else {
    // s8 output rows: 16 channels per 16-byte store
    constexpr int NG = CPL / 16;
    static_assert(CPL % 16 == 0, "s8 kernels need TN >= 64");
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
      const int o = out_row[rb];
      const bool row_ok = o >= 0 && o < p.rows_c;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int ch = ch0 + g * 16;
        const bool ok = row_ok && ch < p.k_out;
        const uint32_t coff = ok ? (uint32_t)((int64_t)o * p.ldc + ch) : kOob;
        v4i src = {0, 0, 0, 0};
        if (p.read_source) {
          const uint32_t doff = ok ? (uint32_t)((int64_t)o * p.ldd + ch) : kOob;
          src = __builtin_amdgcn_raw_buffer_load_b128(rs_d, doff, 0, 0);
        }
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
            const int c = ch + x < p.k_out ? ch + x : 0;
            t = __builtin_fmaf(p.scale[c], (float)a, p.bias[c]);
            if (p.read_source) t = __builtin_fmaf(p.beta, (float)sb[x], t);
          } else if (p.read_source) {
            t = __builtin_fmaf(p.alpha, (float)a, p.beta * (float)sb[x]);
          } else {
            t = p.alpha * (float)a;
          }
          t = apply_act(t, p.act, p.act_alpha);
          ob[x] = (int8_t)f32_to_s8(t);
        }
        __builtin_amdgcn_raw_buffer_store_b128(outv, rs_c, coff, 0, 0);
      }
    }
  }
}

}  // namespace cummhip
