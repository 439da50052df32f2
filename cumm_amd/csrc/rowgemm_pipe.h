// Deeply pipelined variant of the gather-rows GEMM (see rowgemm.h for the data mapping) for
// contractions that fit one channel chunk.
//
// A tile's kernel offsets are walked BW at a time ("steps").  Three cursors run over the set bits
// of the tile mask at different distances ahead of the MFMAs:
//
//     pair-table entries of step p + DA + DI   (4 bytes per row and offset)
//     gathered rows of step p + DA             (straight into MFMA operand registers)
//     weight slices of step p + 1              (registers, parked in LDS at the start of step p+1)
//
// so that up to DA steps of gathered rows are in flight while step p computes, and a tile with
// many offsets costs about one memory round trip per DA steps instead of one per step.  Loads
// complete in issue order, so every step issues its requests oldest-needed-first (weights, then
// pair-table entries, then rows): waiting for what the next step needs never waits for what a
// later step needs.  The register sets form rings that are indexed at compile time (the step
// loop is unrolled by the ring length), because copying a register that a load is still filling
// would wait for the load.  For the same reason the step body is straight-line code: a load that
// is skipped on one path makes the number of outstanding loads path dependent and the compiler
// then waits for all of them; a kernel offset past the end of the tile mask is therefore not
// skipped but loaded through an empty buffer descriptor (every lane out of range, zeros back,
// no memory traffic).
#pragma once
#include <type_traits>
#include <utility>

#include "rowgemm.h"

namespace cummhip {

constexpr int ring_lcm(int a, int b) {
  int l = a;
  while (l % b) l += a;
  return l;
}

// runs f(integral_constant<0>), f(integral_constant<1>), ... until one returns true
template <class F, int... Is>
__device__ __forceinline__ bool run_unrolled(F &f, std::integer_sequence<int, Is...>) {
  return (f(std::integral_constant<int, Is>{}) || ...);
}

template <class T, int NW, int RB, int TN, int KS, bool WT, int BW, int DA, int DI, int DW, bool WIDE = false>
__global__ __launch_bounds__(NW * 64) void rowgemm_pipe_kernel(const RowGemmParams p) {
  using E = Elem<T>;
  using AccV = typename E::AccV;
  constexpr int TM = NW * RB * 16;
  constexpr int NB = TN / 16;
  constexpr int CPL = TN / 4;
  constexpr int PV = E::kPerVec;
  constexpr int SLICE_V = NB * KS * 64;
  constexpr int NT = NW * 64;
  constexpr int RA = DA + 1;        // ring of gathered-row register sets
  constexpr int RI = DI + 1;        // ring of pair-table register sets
  constexpr int UNROLL = ring_lcm(ring_lcm(RA, RI), DW);  // all rings are back at slot 0 after this many steps

  __shared__ v4i lds_w[2][BW * SLICE_V];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 15;
  const int q = lane >> 4;

  const int tile = (int)gridDim.x - 1 - (int)blockIdx.x;  // heaviest tiles first
  const int n0 = blockIdx.y * TN;
  const int pos_base = tile * TM;

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

  int out_row[RB];
  uint32_t key_off[RB];
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

  const uint32_t a_row_bytes = (uint32_t)p.lda * E::kBytes;
  const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(p.A, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(p.W, p.w_bytes);
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(p.gather, p.gather ? p.gather_bytes : 0u);
  const __amdgpu_buffer_rsrc_t rs_none = make_rsrc(p.A, 0u);   // every offset out of range
  const bool has_gather = p.gather != nullptr;

  constexpr int GRAN = TN * 4 * KS;
  constexpr int GPT = (GRAN + NT - 1) / NT;

  // ---- everything about addresses that does not depend on the kernel offset is computed once:
  // the step loop is bound by instruction issue as soon as it recomputes them per step.
  // gathered rows: piece s*4 + q of the row (one 64-byte segment of each row per instruction)
  const uint32_t a_col = (uint32_t)q * 16u;
  bool a_col_ok[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) a_col_ok[s] = (s * 4 + q) * PV < p.c_in;
  // weight granules of this thread: byte offset at kernel offset 0 and LDS slot (16-byte units)
  uint32_t w_voff[GPT];
  int w_slot[GPT];   // non-transposing: slot of the granule; transposing: see park_w
  const uint32_t w_k_bytes = (uint32_t)p.w_stride_k * E::kBytes;
#pragma unroll
  for (int i = 0; i < GPT; ++i) {
    const int id = tid + i * NT;
    w_voff[i] = kOob;
    w_slot[i] = 0;
    if constexpr (!WT) {
      const int n_local = id / (4 * KS), g = id % (4 * KS);
      const int n = n0 + n_local, e = g * PV;
      if (id < GRAN && n < p.k_out && e < p.c_in)
        w_voff[i] = (uint32_t)((int64_t)n * p.w_stride_n + e) * E::kBytes;
      const int qo = n_local / CPL, rem = n_local % CPL, nb = rem >> 2, r = rem & 3, qq = g % 4;
      // the low bits are XOR-swizzled so that the staging writes of a wave spread over all banks
      w_slot[i] = (nb * KS + g / 4) * 64 + qq * 16 + ((qo * 4 + r) ^ (qq << 2) ^ (nb & 3));
    } else {
      constexpr int NG = TN / PV;
      const int n = n0 + (id % NG) * PV, e = id / NG;
      if (id < GRAN && n < p.k_out && e < p.c_in)
        w_voff[i] = (uint32_t)((int64_t)e * p.w_stride_c + n) * E::kBytes;
    }
  }
  // LDS read position of this lane inside a 64-slot fragment, one per swizzle variant (nb & 3)
  int rd_slot[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) rd_slot[v] = lane ^ ((q << 2) ^ v);

  // slot of (output channel n_local, contraction piece g) for the transposing stage
  auto lds_slot = [&](int n_local, int g) -> int {
    const int qo = n_local / CPL;
    const int rem = n_local % CPL;
    const int nb = rem >> 2;
    const int r = rem & 3;
    const int qq = g % 4;
    return (nb * KS + g / 4) * 64 + qq * 16 + ((qo * 4 + r) ^ (qq << 2) ^ (nb & 3));
  };

  // register rings
  int idx[RI][BW][RB];
  v4i afrag[RA][BW][RB][KS];
  v4i wreg[DW][BW][GPT];   // weight slices of steps p .. p + DW - 1
  // per-step scalars travel with the ring slots
  int k_of_a[RA][BW];        // offsets whose rows sit in afrag[slot]
  uint64_t any_a[RA][BW][RB];

  int koff1[BW];
  // cursors over the set bits of the tile mask
  uint32_t rem_i = kmask, rem_a = kmask, rem_w = kmask;
  auto take = [&](uint32_t &rem, int (&ko)[BW]) {
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      ko[j] = rem ? __builtin_ctz(rem) : -1;
      if (rem) rem &= rem - 1;
    }
  };

  const uint32_t g_k_bytes = (uint32_t)p.n_idx * 4u;
  auto issue_idx = [&](int (&dst)[BW][RB]) {
    int ko[BW];
    take(rem_i, ko);
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      const bool live = ko[j] >= 0 && has_gather;
      const __amdgpu_buffer_rsrc_t rs = live ? rs_g : rs_none;
      const uint32_t soff = live ? (uint32_t)ko[j] * g_k_bytes : 0u;   // row of the table
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int v = __builtin_amdgcn_raw_buffer_load_b32(rs, key_off[rb], soff, 0);
        dst[j][rb] = has_gather ? v : (int)(key_off[rb] >> 2);
      }
    }
  };

  auto issue_a = [&](const int (&src)[BW][RB], v4i (&dst)[BW][RB][KS], int (&kdst)[BW],
                     uint64_t (&anyd)[BW][RB]) {
    take(rem_a, kdst);
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      const bool live = kdst[j] >= 0;
      const __amdgpu_buffer_rsrc_t rs = live ? rs_a : rs_none;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int v = src[j][rb];
        const bool ok = key_ok[rb] && v >= 0 && v < p.rows_a;
        anyd[j][rb] = live ? __ballot(ok) : 0;
        const uint32_t row = (uint32_t)v * a_row_bytes + a_col;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          // branch-free select (a ?: here is turned into two loads under complementary masks)
          const uint32_t keep = 0u - (uint32_t)(ok && a_col_ok[s]);
          dst[j][rb][s] = __builtin_amdgcn_raw_buffer_load_b128(
              rs, ((row + (uint32_t)(s * 64)) & keep) | (kOob & ~keep), 0, 0);
        }
      }
    }
  };

  auto issue_w = [&](v4i (&wdst)[BW][GPT]) {
    int ko[BW];
    take(rem_w, ko);
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      const bool live = ko[j] >= 0;
      const __amdgpu_buffer_rsrc_t rs = live ? rs_w : rs_none;
      const uint32_t soff = live ? (uint32_t)ko[j] * w_k_bytes : 0u;
#pragma unroll
      for (int i = 0; i < GPT; ++i) wdst[j][i] = __builtin_amdgcn_raw_buffer_load_b128(rs, w_voff[i], soff, 0);
    }
  };

  auto park_w = [&](int buf, const int (&kcur)[BW], const v4i (&wsrc)[BW][GPT]) {
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      v4i *stage = &lds_w[buf][j * SLICE_V];
      if constexpr (!WT) {
#pragma unroll
        for (int i = 0; i < GPT; ++i)
          if (tid + i * NT < GRAN) stage[w_slot[i]] = wsrc[j][i];
      } else {
        constexpr int NG = TN / PV;
#pragma unroll
        for (int i = 0; i < GPT; ++i) {
          const int id = tid + i * NT;
          if (id < GRAN) {
            const int c_local = id / NG;
            const int ng = id % NG;
            const int g = c_local / PV;
            const int jj = c_local % PV;
            if constexpr (E::kBytes == 2) {
              uint16_t *dst = reinterpret_cast<uint16_t *>(stage);
              const uint16_t *src = reinterpret_cast<const uint16_t *>(&wsrc[j][i]);
#pragma unroll
              for (int x = 0; x < 8; ++x) dst[lds_slot(ng * 8 + x, g) * 8 + jj] = src[x];
            } else {
              uint8_t *dst = reinterpret_cast<uint8_t *>(stage);
              const uint8_t *src = reinterpret_cast<const uint8_t *>(&wsrc[j][i]);
#pragma unroll
              for (int x = 0; x < 16; ++x) dst[lds_slot(ng * 16 + x, g) * 16 + jj] = src[x];
            }
          }
        }
      }
    }
  };

  if (kmask != 0 && __builtin_popcount(kmask) <= BW) {
    // ---- a tile with a single step (the common case with sorted masks): nothing to pipeline,
    // so request exactly what is needed, once, and do not pay for the speculative ring fills
    take(rem_w, koff1);
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      if (koff1[j] < 0) continue;
      const uint32_t soff = (uint32_t)koff1[j] * w_k_bytes;
#pragma unroll
      for (int i = 0; i < GPT; ++i) wreg[0][j][i] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, w_voff[i], soff, 0);
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        idx[0][j][rb] = has_gather ? __builtin_amdgcn_raw_buffer_load_b32(rs_g, key_off[rb], (uint32_t)koff1[j] * g_k_bytes, 0)
                                   : (int)(key_off[rb] >> 2);
    }
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      if (koff1[j] < 0) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) any_a[0][j][rb] = 0;
        continue;
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const int v = idx[0][j][rb];
        const bool ok = key_ok[rb] && v >= 0 && v < p.rows_a;
        any_a[0][j][rb] = __ballot(ok);
        const uint32_t row = (uint32_t)v * a_row_bytes + a_col;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const uint32_t keep = 0u - (uint32_t)(ok && a_col_ok[s]);
          afrag[0][j][rb][s] = __builtin_amdgcn_raw_buffer_load_b128(
              rs_a, ((row + (uint32_t)(s * 64)) & keep) | (kOob & ~keep), 0, 0);
        }
      }
    }
    park_w(0, koff1, wreg[0]);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < BW; ++j) {
      if (koff1[j] < 0) continue;
      uint64_t any_j = 0;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) any_j |= any_a[0][j][rb];
      if (any_j == 0) continue;
      const v4i *stage = &lds_w[0][j * SLICE_V];
      v4i wf[NB][KS];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int s = 0; s < KS; ++s) wf[nb][s] = stage[(nb * KS + s) * 64 + rd_slot[nb & 3]];
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        if (RB > 1 && any_a[0][j][rb] == 0) continue;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int s = 0; s < KS; ++s) acc[rb][nb] = E::mfma(wf[nb][s], afrag[0][j][rb][s], acc[rb][nb]);
      }
    }
  } else if (kmask != 0) {
    // ---- prologue: fill the pipeline
#pragma unroll
    for (int i = 0; i < DW; ++i) issue_w(wreg[i]);    // weights of steps 0 .. DW-1
#pragma unroll
    for (int i = 0; i < RI; ++i) issue_idx(idx[i]);   // pair-table entries of steps 0 .. DI
    // rows of steps 0 .. DA-1 need entries of steps 0 .. DA-1; the entry ring holds DI+1 steps, so
    // refill it as it is consumed
#pragma unroll
    for (int s = 0; s < DA; ++s) {
      issue_a(idx[s % RI], afrag[s % RA], k_of_a[s % RA], any_a[s % RA]);
      issue_idx(idx[s % RI]);
    }
    // ---- steady state, unrolled so that every ring slot is a compile-time index
    int buf = 0;
    auto step = [&](auto uc) -> bool {
      constexpr int u = decltype(uc)::value;
      constexpr int sa = u % RA;             // slot whose rows this step consumes
      constexpr int sn = (u + DA) % RA;      // slot that receives the rows of step p + DA
      constexpr int si = (u + DA) % RI;      // entries of step p + DA (then refilled)
      int kcur[BW];
#pragma unroll
      for (int j = 0; j < BW; ++j) kcur[j] = k_of_a[sa][j];
      park_w(buf, kcur, wreg[u % DW]);   // waits for this step's weights only
      issue_w(wreg[u % DW]);             // weights of step p + DW, first: they are needed soonest
      issue_a(idx[si], afrag[sn], k_of_a[sn], any_a[sn]);   // rows of step p + DA
      issue_idx(idx[si]);                // entries of step p + DA + DI + 1
      __syncthreads();
#pragma unroll
      for (int j = 0; j < BW; ++j) {
        uint64_t any_j = 0;
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) any_j |= any_a[sa][j][rb];
        if (any_j == 0) continue;   // no row of this wave has a pair at this offset
        const v4i *stage = &lds_w[buf][j * SLICE_V];
        v4i wf[NB][KS];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int s = 0; s < KS; ++s) wf[nb][s] = stage[(nb * KS + s) * 64 + rd_slot[nb & 3]];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          if (RB > 1 && any_a[sa][j][rb] == 0) continue;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int s = 0; s < KS; ++s) acc[rb][nb] = E::mfma(wf[nb][s], afrag[sa][j][rb][s], acc[rb][nb]);
        }
      }
      buf ^= 1;
      // the next step's first offset is absent when the tile mask is exhausted
      return k_of_a[(u + 1) % RA][0] < 0;
    };
    while (!run_unrolled(step, std::make_integer_sequence<int, UNROLL>{})) {
    }
  }

  // ---- epilogue (as rowgemm_kernel)
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
    constexpr int NG = CPL / 8;
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
          float t = p.read_source ? __builtin_fmaf(p.alpha, a, p.beta * E::to_float(sh[x])) : p.alpha * a;
          t = apply_act(t, p.act, p.act_alpha);
          oh[x] = E::from_float(t);
        }
        __builtin_amdgcn_raw_buffer_store_b128(outv, rs_c, coff, 0, 0);
      }
    }
  } else {
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
