// Dense GEMM for operands that are both contiguous along the contraction,
//   D[m][n] = epilogue( sum_k Y[m][k] * X[n][k] ),   k a multiple of the step,
// streamed through an LDS ring with direct-to-LDS buffer loads (see lds_dma.h and rowgemm_lds.h
// for the mechanism: hidden loads, hand-counted waits, fence-less barrier, XOR-permuted 16-byte
// chunks applied on the global side).
//
// What differs from tilegemm.h, and why:
//   * the wave tile (RBW x NBW blocks of 16 x 16) and the step depth are template parameters;
//     per k-step of 32 a wave reads (RBW + NBW) KB of fragments for RBW*NBW MFMAs, so larger wave
//     tiles need fewer LDS bytes per MFMA (the chip lowers its clock under MFMA load, what
//     counts is work per MFMA, not only cycles);
//   * nothing passes through registers on the way in, no LDS stores, one barrier per step, the
//     loads of step s + NS - 1 are in flight while step s computes;
//   * X rows sit in LDS in the order that gives a lane 4*NBW consecutive output columns
//     (row nb*16 + i of a wave's slab holds column (i/4)*4*NBW + nb*4 + i%4): 16-byte stores;
//   * workgroup numbers are mapped to tiles so that the workgroups that share an XCD (numbers
//     w, w + 8, ...) work on neighbouring tiles: 8 tile rows x all tile columns at a time, each
//     operand panel is fetched into that XCD's L2 once per group.
#pragma once
#include "lds_dma.h"
#include "tilegemm.h"

namespace cummhip {

template <class T, int WM, int WN, int RBW, int NBW, int KS, int NS>
__global__ __launch_bounds__(WM *WN * 64) void densegemm_lds_kernel(const TileGemmParams p, int tiles_m, int tiles_n) {
  using E = Elem<T>;
  using AccV = typename E::AccV;
  constexpr int NT = WM * WN * 64;
  constexpr int TM = WM * RBW * 16;
  constexpr int TN = WN * NBW * 16;
  constexpr int PV = E::kPerVec;
  constexpr int LPR = 4 * KS;              // 16-byte chunks per row and step
  constexpr int RPI = 64 / LPR;            // rows per load instruction
  constexpr int IPY = TM * LPR / NT;       // load instructions per wave and step
  constexpr int IPX = TN * LPR / NT;
  static_assert(IPY >= 1 && IPX >= 1, "tile too small for the workgroup");
  constexpr int Y_V = TM * LPR;            // 16-byte vectors of the Y part of a stage
  constexpr int STAGE_V = (TM + TN) * LPR;
  constexpr int L = NS - 1;                // steps the loads run ahead
  constexpr int PER_STEP = IPY + IPX;
  constexpr int WAIT_STEP = (L - 1) * PER_STEP;   // loads issued after those of step s when it starts
  static_assert(WAIT_STEP < 64, "too many loads in flight for the counter");
  constexpr int BK = KS * 64 / E::kBytes;  // contraction elements per step
  constexpr uint32_t kOob = 0x80000000u;

  __shared__ v4i ring[NS * STAGE_V];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int m = lane & 15, q = lane >> 4;

  // ---- tile of this workgroup
  int logical = blockIdx.x;
  const int nwg = gridDim.x;
  if (nwg % 8 == 0) logical = (blockIdx.x % 8) * (nwg / 8) + blockIdx.x / 8;
  constexpr int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int g = logical / per_group, r = logical % per_group;
  const int rows_here = tiles_m - g * GROUP < GROUP ? tiles_m - g * GROUP : GROUP;
  const int tile_m = g * GROUP + r % rows_here, tile_n = r / rows_here;
  const int m0 = tile_m * TM, n0 = tile_n * TN;

  // ---- loader role
  const int lrow = lane / LPR, lchunk = lane % LPR;
  auto swz = [](int row) { return KS == 1 ? (row >> 1) & 3 : ((row * KS) >> 2) & (LPR - 1); };
  uint32_t y_voff[IPY], x_voff[IPX];
#pragma unroll
  for (int t = 0; t < IPY; ++t) {
    const int row = (wave * IPY + t) * RPI + lrow;
    const int gm = m0 + row;
    const int c = lchunk ^ swz(row);
    y_voff[t] = gm < p.m ? (uint32_t)((int64_t)gm * p.ldy * E::kBytes) + (uint32_t)c * 16u : kOob;
  }
#pragma unroll
  for (int t = 0; t < IPX; ++t) {
    const int rho = (wave * IPX + t) * RPI + lrow;      // LDS row, fragment order
    const int i = rho & 15, nb = (rho >> 4) % NBW, wq = rho / (16 * NBW);
    const int n = n0 + wq * (16 * NBW) + (i >> 2) * (4 * NBW) + nb * 4 + (i & 3);
    const int c = lchunk ^ swz(rho);
    x_voff[t] = n < p.n ? (uint32_t)((int64_t)n * p.ldx * E::kBytes) + (uint32_t)c * 16u : kOob;
  }
  const uint32_t y_bytes = (uint32_t)(((int64_t)(p.m - 1) * p.ldy + p.k) * E::kBytes);
  const uint32_t x_bytes = (uint32_t)(((int64_t)(p.n - 1) * p.ldx + p.k) * E::kBytes);
  const int steps = p.k / BK;

  // ---- reader role: fragment slots (16-byte units) inside a stage
  int y_rd[KS], x_rd[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int slot = m * LPR + ((s * 4 + q) ^ swz(m));
    y_rd[s] = wm * (RBW * 16) * LPR + slot;
    x_rd[s] = Y_V + wn * (NBW * 16) * LPR + slot;
  }

  AccV acc[RBW][NBW];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb) acc[rb][nb] = AccV{0, 0, 0, 0};

  const uint32_t ring_at = lds_addr(ring);
  auto issue = [&](int s, int stage) __attribute__((always_inline)) {
    // a step past the end is fetched through descriptors without records: zeros, no traffic,
    // the same number of loads in flight
    const bool live = s < steps;
    const v4i rs_y = rsrc_words(p.Y, live ? y_bytes : 0u);
    const v4i rs_x = rsrc_words(p.X, live ? x_bytes : 0u);
    const uint32_t soff = (uint32_t)__builtin_amdgcn_readfirstlane(s * BK * E::kBytes);
    const uint32_t st = ring_at + (uint32_t)__builtin_amdgcn_readfirstlane(stage * STAGE_V * 16);
#pragma unroll
    for (int t = 0; t < IPY; ++t) dma_b128(rs_y, st + (wave * IPY + t) * 1024, y_voff[t], soff);
#pragma unroll
    for (int t = 0; t < IPX; ++t) dma_b128(rs_x, st + Y_V * 16 + (wave * IPX + t) * 1024, x_voff[t], soff);
  };

  for (int s = 0; s < L; ++s) issue(s, s);
  int cs = 0, ls = L;   // stage computed, stage loaded (the one the previous step computed)
  for (int s = 0; s < steps; ++s) {
    wait_vmcnt<WAIT_STEP>();
    lds_barrier();
    const v4i *st = ring + cs * STAGE_V;
    v4i yf[RBW][KS], xf[NBW][KS];
#pragma unroll
    for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
      for (int k = 0; k < KS; ++k) xf[nb][k] = st[x_rd[k] + nb * 16 * LPR];
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
      for (int k = 0; k < KS; ++k) yf[rb][k] = st[y_rd[k] + rb * 16 * LPR];
    issue(s + L, ls);
    cs = cs + 1 == NS ? 0 : cs + 1;
    ls = ls + 1 == NS ? 0 : ls + 1;
#pragma unroll
    for (int k = 0; k < KS; ++k)
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
        for (int nb = 0; nb < NBW; ++nb) acc[rb][nb] = E::mfma(xf[nb][k], yf[rb][k], acc[rb][nb]);
  }
  wait_vmcnt<0>();

  // ---- epilogue: lane (q, m) holds, for each of its rows, columns ch0 .. ch0 + 4*NBW - 1
  constexpr int CPLW = 4 * NBW;
  static_assert(E::kBytes == 2 && CPLW % 8 == 0, "two-byte outputs, whole 16-byte pieces");
  const bool read_src = p.beta != 0.0f;
  const int ch0 = n0 + wn * (NBW * 16) + q * CPLW;
  uint16_t *cbase = reinterpret_cast<uint16_t *>(p.C);
  const uint16_t *dbase = reinterpret_cast<const uint16_t *>(p.D);
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int mm = m0 + (wm * RBW + rb) * 16 + m;
    if (mm >= p.m) continue;
#pragma unroll
    for (int gi = 0; gi < CPLW / 8; ++gi) {
      const int nn = ch0 + gi * 8;
      if (nn >= p.n) continue;
      v4i sv = {0, 0, 0, 0};
      if (read_src) sv = *reinterpret_cast<const v4i *>(dbase + (int64_t)mm * p.ldd + nn);
      const uint16_t *sh = reinterpret_cast<const uint16_t *>(&sv);
      v4i ov;
      uint16_t *oh = reinterpret_cast<uint16_t *>(&ov);
#pragma unroll
      for (int x = 0; x < 8; ++x) {
        const float a = acc[rb][gi * 2 + (x >> 2)][x & 3];
        float t = read_src ? __builtin_fmaf(p.alpha, a, p.beta * E::to_float(sh[x])) : p.alpha * a;
        t = apply_act(t, p.act, p.act_alpha);
        oh[x] = E::from_float(t);
      }
      *reinterpret_cast<v4i *>(cbase + (int64_t)mm * p.ldc + nn) = ov;
    }
  }
}

}  // namespace cummhip
