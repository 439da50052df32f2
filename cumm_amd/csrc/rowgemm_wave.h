// Gather-GEMM-scatter with ONE weight matrix (matmul2 with ShuffleAC: C[c_inds[i]] = act(alpha *
// A[a_inds[i]] @ op(B) + beta * D[c_inds[i]]); the reference's gemm_kernel with gather iterators,
// cumm/gemm/kernel.py:585-939) for contractions of at most 128 two-byte elements.
//
// Why a kernel of its own: with a single weight matrix nothing has to be staged per step.  The
// matrix (at most 64 channels x 256 bytes per column block) goes into MFMA operand registers once
// per wave - through LDS, in the row order that gives a lane 16 consecutive output channels -, and
// after that a wave works alone: it gathers 16 rows straight into operand registers (lane (q, m)
// loads bytes 16 q .. 16 q + 15 of each 64-byte piece of row m), multiplies, and scatters 16-byte
// pieces.  No LDS traffic per row, no barrier after the first, no ring: what bounds the occupancy
// is registers (four to five waves per SIMD), so one launch has every row block of a 150 k-pair
// problem in flight in two to three rounds, against 1.5 generations of 128-row tiles with three
// workgroups per CU in the LDS-streaming kernel (13.2 us against 14.1 us on 150 k pairs of 64
// channels: 58.8 MB at 4.4 TB/s, where a plain gather of 128-byte rows reaches about 6).
// Two row blocks per trip are requested together, indices first, rows and source rows next.
// Taken for up to 64 output channels (grid.y = 1 then; the code below handles more column blocks,
// each gathering the rows again).
#pragma once
#include "lds_dma.h"
#include "rowgemm.h"

namespace cummhip {

// T: element tag (two-byte elements); KS: 64-byte pieces per row (contraction <= 32 * KS elements).
// WT false: B stored [n, k] (w_stride_c == 1); WT true: B stored [k, n] (w_stride_n == 1).
// WIDE: f32 outputs (as store_wide_piece in rowgemm.h).  grid.y = 64-channel column blocks.
template <class T, int KS, bool WT, bool WIDE>
__global__ __launch_bounds__(256) void rowgemm_wave_kernel(const RowGemmParams p) {
  using E = Elem<T>;
  static_assert(E::kBytes == 2, "two-byte elements");
  constexpr int NB = 4;                 // 16-channel blocks of the column block
  constexpr int KE = KS * 32;           // contraction elements held in LDS per channel
  constexpr int U = 2;                  // row blocks per trip
  __shared__ __attribute__((aligned(16))) uint16_t wl[64 * KE];   // [fragment-order row][contraction]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 15, q = lane >> 4;
  const int n0 = (int)blockIdx.y * 64;

  // ---- row blocks of 16: this wave takes blocks gw, gw + waves, ...; the row numbers of its first
  // trip are requested before anything else (their round trip runs next to the weights')
  const bool has_gather = p.gather != nullptr, has_rows = p.out_rows != nullptr;
  const __amdgpu_buffer_rsrc_t rs_g = make_rsrc(p.gather, has_gather ? (uint32_t)p.n_pos * 4u : 0u);
  const __amdgpu_buffer_rsrc_t rs_o = make_rsrc(p.out_rows, has_rows ? (uint32_t)p.n_pos * 4u : 0u);
  const __amdgpu_buffer_rsrc_t rs_a = make_rsrc(p.A, p.a_bytes);
  const __amdgpu_buffer_rsrc_t rs_c = make_rsrc(p.C, p.c_bytes);
  const __amdgpu_buffer_rsrc_t rs_d = make_rsrc(p.D, p.read_source ? p.d_bytes : 0u);
  const int n_blocks = (p.n_pos + 15) >> 4;
  const int waves = (int)gridDim.x * 4;
  const int ch0 = n0 + q * 16;
  const uint32_t a_row_bytes = (uint32_t)p.lda * 2u;
  const int first_block = (int)blockIdx.x * 4 + wave;
  auto row_numbers = [&](int b0, int (&arow)[U], int (&orow)[U]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = (b0 + u * waves) * 16 + m;
      const bool in = b0 + u * waves < n_blocks && r < p.n_pos;
      const uint32_t off = in ? (uint32_t)r * 4u : kOob;
      const int g = __builtin_amdgcn_raw_buffer_load_b32(rs_g, off, 0, 0);
      const int o = __builtin_amdgcn_raw_buffer_load_b32(rs_o, off, 0, 0);
      arow[u] = in ? (has_gather ? g : r) : -1;
      orow[u] = in ? (has_rows ? o : r) : -1;
    }
  };
  int arow0[U], orow0[U];
  row_numbers(first_block, arow0, orow0);

  // ---- the weights of this column block: LDS row nb * 16 + i holds output channel
  // n0 + (i / 4) * 16 + nb * 4 + i % 4, so that the MFMA result rows 4 q .. 4 q + 3 of block nb are
  // channels n0 + 16 q + 4 nb .. + 3: a lane ends up with 16 consecutive channels of its row
  const __amdgpu_buffer_rsrc_t rs_w = make_rsrc(p.W, p.w_bytes);
  if constexpr (!WT) {
    constexpr int CPR = KE / 8;         // 16-byte chunks per channel
#pragma unroll
    for (int it = 0; it < (64 * CPR) / 256; ++it) {
      const int v = it * 256 + tid;
      const int rho = v / CPR, c = v % CPR;
      const int i = rho & 15, nb = rho >> 4;
      const int n = n0 + (i >> 2) * 16 + nb * 4 + (i & 3);
      const bool ok = n < p.k_out && c * 8 < p.c_in;
      const v4i w = __builtin_amdgcn_raw_buffer_load_b128(
          rs_w, ok ? (uint32_t)((int64_t)n * p.w_stride_n * 2) + (uint32_t)c * 16u : kOob, 0, 0);
      *reinterpret_cast<v4i *>(&wl[rho * KE + c * 8]) = w;
    }
  } else {
    // eight channels of one contraction row per load, parked transposed with 16-bit stores
#pragma unroll
    for (int it = 0; it < (KE * 8) / 256; ++it) {
      const int v = it * 256 + tid;
      const int k = v >> 3, g = v & 7;
      const int n = n0 + g * 8;
      const bool ok = n < p.k_out && k < p.c_in;
      const v4i w = __builtin_amdgcn_raw_buffer_load_b128(
          rs_w, ok ? (uint32_t)(((int64_t)k * p.w_stride_c + n) * 2) : kOob, 0, 0);
      const uint16_t *wh = reinterpret_cast<const uint16_t *>(&w);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int cl = g * 8 + e;                                   // channel inside the column block
        const int rho = ((cl & 15) >> 2) * 16 + (cl >> 4) * 4 + (cl & 3);
        wl[rho * KE + k] = wh[e];
      }
    }
  }
  __syncthreads();
  v4i wf[NB][KS];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int s = 0; s < KS; ++s) wf[nb][s] = *reinterpret_cast<const v4i *>(&wl[(nb * 16 + m) * KE + (s * 4 + q) * 8]);

  for (int b0 = first_block; b0 < n_blocks; b0 += waves * U) {
    int arow[U], orow[U];
    if (b0 == first_block) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        arow[u] = arow0[u];
        orow[u] = orow0[u];
      }
    } else {
      row_numbers(b0, arow, orow);
    }
    // a lane's 16 output channels of a row: two 16-byte pieces of two-byte outputs, four of f32
    constexpr int NP = WIDE ? 4 : 2, CPP = 16 / NP, OB = WIDE ? 4 : 2;   // pieces, channels per piece, bytes per output
    v4i af[U][KS];
    v4i src[U][NP];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bool a_ok = (uint32_t)arow[u] < (uint32_t)p.rows_a;
#pragma unroll
      for (int s = 0; s < KS; ++s)
        af[u][s] = __builtin_amdgcn_raw_buffer_load_b128(
            rs_a, a_ok && s * 32 + q * 8 < p.c_in ? (uint32_t)arow[u] * a_row_bytes + (uint32_t)(s * 64 + q * 16) : kOob, 0, 0);
      const bool o_ok = orow[u] >= 0 && orow[u] < p.rows_c;
#pragma unroll
      for (int g = 0; g < NP; ++g) {
        const int ch = ch0 + g * CPP;
        src[u][g] = __builtin_amdgcn_raw_buffer_load_b128(
            rs_d, o_ok && ch < p.k_out ? (uint32_t)((int64_t)orow[u] * p.ldd + ch) * (uint32_t)OB : kOob, 0, 0);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      v4f acc[NB];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) acc[nb] = v4f{0, 0, 0, 0};
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = E::mfma(wf[nb][s], af[u][s], acc[nb]);
      const int o = orow[u];
      const bool row_ok = o >= 0 && o < p.rows_c;
      if constexpr (WIDE) {
        // (the f32 branch of store_wide_piece, with the source rows requested above)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int ch = ch0 + nb * 4;
          const v4f sf = __builtin_bit_cast(v4f, src[u][nb]);
          v4f of;
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            const float t = p.read_source ? __builtin_fmaf(p.alpha, acc[nb][x], p.beta * sf[x]) : p.alpha * acc[nb][x];
            of[x] = apply_act(t, p.act, p.act_alpha);
          }
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i, of), rs_c,
                                                 row_ok && ch < p.k_out ? (uint32_t)((int64_t)o * p.ldc + ch) * 4u : kOob, 0, 0);
        }
      } else {
#pragma unroll
        for (int g = 0; g < 2; ++g) {
          const int ch = ch0 + g * 8;
          const bool ok = row_ok && ch < p.k_out;
          const uint16_t *sh = reinterpret_cast<const uint16_t *>(&src[u][g]);
          v4i outv;
          uint16_t *oh = reinterpret_cast<uint16_t *>(&outv);
#pragma unroll
          for (int x = 0; x < 8; ++x) {
            const float a = acc[g * 2 + (x >> 2)][x & 3];
            float t = p.read_source ? __builtin_fmaf(p.alpha, a, p.beta * E::to_float(sh[x])) : p.alpha * a;
            t = apply_act(t, p.act, p.act_alpha);
            oh[x] = E::from_float(t);
          }
          __builtin_amdgcn_raw_buffer_store_b128(outv, rs_c, ok ? (uint32_t)((int64_t)o * p.ldc + ch) * 2u : kOob, 0, 0);
        }
      }
    }
  }
}

}  // namespace cummhip
