// Instantiations of the LDS-tiled GEMM for one element type (selected with -DCUMM_ELEM=...).
#include "launch.h"
#include "densegemm_lds.h"

namespace cummhip {

#define CUMM_CAT_(a, b) a##b
#define CUMM_CAT(a, b) CUMM_CAT_(a, b)

// -DCUMM_WIDE=1 builds the tiled kernels with four-byte outputs (s32 / f32) under the name
// launch_tilegemm_wide_<type>, in a translation unit of its own (and nothing else)
#ifndef CUMM_WIDE
#define CUMM_WIDE 0
#endif
constexpr bool kWide = CUMM_WIDE != 0;
#if CUMM_WIDE
#define CUMM_LAUNCH_NAME CUMM_CAT(launch_tilegemm_wide_, CUMM_NAME)
#else
#define CUMM_LAUNCH_NAME CUMM_CAT(launch_tilegemm_, CUMM_NAME)
#endif

template <class T, int BM, int BN>
static hipError_t launch_xy(bool xk, bool yk, const TileGemmParams &p, dim3 grid, hipStream_t s) {
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;
  if (xk && yk) hipLaunchKernelGGL((tilegemm_kernel<T, true, true, BM, BN, 1, kWide>), grid, dim3(256), 0, s, p);
  else if (xk && !yk) hipLaunchKernelGGL((tilegemm_kernel<T, true, false, BM, BN, 1, kWide>), grid, dim3(256), 0, s, p);
  else if (!xk && yk) hipLaunchKernelGGL((tilegemm_kernel<T, false, true, BM, BN, 1, kWide>), grid, dim3(256), 0, s, p);
  else hipLaunchKernelGGL((tilegemm_kernel<T, false, false, BM, BN, 1, kWide>), grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

// Plain GEMM with both operands contiguous along the contraction, two-byte elements, shapes
// the LDS-ring kernel takes without a remainder in k and with 16-byte output pieces.  Its result
// does not depend on the tile (one fp32 sum over k in ascending order per element either way).
// Measured on 4096^3 f16 (TFLOP/s): 256 x 256 x 32 per step with 2 x 4 waves of 128 x 64 and
// three stages 1089, the same with 4 x 2 waves of 64 x 128 954, with four stages 1066, with 64
// per step and two stages 1011; 128 x 128 x 64 with 2 x 2 waves and two stages 966; 256 x 128 x 32
// with three stages 902; the register-staged kernel 583.
template <class T, int WM, int WN, int RBW, int NBW, int KS, int NS>
static hipError_t launch_dense_ring_as(const TileGemmParams &p, hipStream_t s) {
  constexpr int TM = WM * RBW * 16, TN = WN * NBW * 16;
  if (!counted_waits_hold<densegemm_lds_kernel<T, WM, WN, RBW, NBW, KS, NS>>()) return hipErrorNotSupported;
  const int tiles_m = (p.m + TM - 1) / TM, tiles_n = (p.n + TN - 1) / TN;
  hipLaunchKernelGGL((densegemm_lds_kernel<T, WM, WN, RBW, NBW, KS, NS>), dim3((unsigned)(tiles_m * tiles_n)),
                     dim3(WM * WN * 64), 0, s, p, tiles_m, tiles_n);
  return hipGetLastError();
}

template <class T>
static bool launch_dense_ring(const TileGemmParams &p, hipStream_t s, hipError_t *err) {
  if constexpr (Elem<T>::kBytes != 2) {
    return false;
  } else {
    const auto al16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const bool ok = p.kv == 1 && p.split_k == 1 && !p.x_gather && !p.y_gather && !p.red_mask &&
                    p.k >= 64 && p.k % 64 == 0 && p.n % 8 == 0 && p.ldx % 8 == 0 && p.ldy % 8 == 0 &&
                    p.ldc % 8 == 0 && p.ldd % 8 == 0 && al16(p.X) && al16(p.Y) && al16(p.C) && al16(p.D) &&
                    ((int64_t)(p.m - 1) * p.ldy + p.k) * 2 < ((int64_t)1 << 31) &&
                    ((int64_t)(p.n - 1) * p.ldx + p.k) * 2 < ((int64_t)1 << 31);
    if (!ok) return false;
    const int64_t big_tiles = (int64_t)((p.m + 255) / 256) * ((p.n + 255) / 256);
    const int64_t mid_tiles = (int64_t)((p.m + 127) / 128) * ((p.n + 127) / 128);
    if (big_tiles >= 256) *err = launch_dense_ring_as<T, 2, 4, 8, 4, 1, 3>(p, s);       // a tile per CU at least
    else if (mid_tiles >= 64) *err = launch_dense_ring_as<T, 2, 2, 4, 4, 2, 2>(p, s);
    else return false;
    return *err != hipErrorNotSupported;     // (the register-staged kernel takes over)
  }
}

hipError_t CUMM_LAUNCH_NAME(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid, hipStream_t s) {
  using T = CUMM_ELEM;
  if constexpr (!kWide) {
    if (xk && yk) {
      hipError_t err = hipSuccess;
      if (launch_dense_ring<T>(p, s, &err)) return err;
    }
  }
  if (tm == 64 && tn == 64) return launch_xy<T, 2, 2>(xk, yk, p, grid, s);
  if (tm == 128 && tn == 128) return launch_xy<T, 4, 4>(xk, yk, p, grid, s);
  return hipErrorInvalidValue;
}

#if !defined(CUMM_NO_WGRAD_ATOMIC) && !CUMM_WIDE
hipError_t CUMM_CAT(launch_wgrad_atomic_, CUMM_NAME)(const WgradParams &p, const WgradPrepareParams &pre,
                                                     const WgradFinalizeParams &f, hipStream_t s) {
  using T = CUMM_ELEM;
  const int groups = (p.num_red + p.tiles_per_wg - 1) / p.tiles_per_wg;
  // both channel counts above 64: units of 128 x 128 channels (one gather of the full rows)
  const bool wide = p.live_list != nullptr && p.K > 64 && p.C > 64;
  const int cpu_ = wide ? 128 : 64;   // channels per unit block
  const int kblocks = (p.K + cpu_ - 1) / cpu_, cblocks = (p.C + cpu_ - 1) / cpu_;
  if (groups == 0 || p.kv == 0) return hipSuccess;
  hipError_t e;
  const bool units_ok = wide ? counted_waits_hold<wgrad_units_kernel<T, 2, 2, 1>>() : counted_waits_hold<wgrad_units_kernel<T, 1, 1, 2>>();
  if (p.live_list != nullptr && !units_ok) return hipErrorNotSupported;
  if (p.live_list != nullptr) {
    // lists + zeroed image, then a resident grid that walks the units
    static int resident_of[2][16] = {};
    int dev = 0;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    int &resident = resident_of[wide ? 1 : 0][dev & 15];
    if (resident == 0) {
      int cus = 0, per_cu = 0;
      e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e == hipSuccess)
        e = wide ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, wgrad_units_kernel<T, 2, 2, 1>, 256, 0)
                 : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, wgrad_units_kernel<T, 1, 1, 2>, 256, 0);
      if (e != hipSuccess) return e;
      resident = cus * per_cu > 0 ? cus * per_cu : 1;
    }
    hipLaunchKernelGGL(wgrad_prepare_kernel, dim3(p.kv + 256), dim3(256), 0, s, pre);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // With several 64 x 64 channel blocks a unit either takes one of them (more units: small
    // inputs) or walks them all on one set of pair lists (the centre offset alone then gives
    // `groups` units: enough when that fills the device).
    WgradParams q = p;
    q.merge_blocks = kblocks * cblocks > 1 && groups >= resident ? 1 : 0;
    // never more workgroups than units can exist
    const long long max_units = ((long long)groups * p.kv + p.kv) * (q.merge_blocks ? 1 : kblocks * cblocks);
    const dim3 units_grid((unsigned)(max_units < resident ? max_units : resident));
    if (wide) hipLaunchKernelGGL((wgrad_units_kernel<T, 2, 2, 1>), units_grid, dim3(256), 0, s, q);
    else hipLaunchKernelGGL((wgrad_units_kernel<T, 1, 1, 2>), units_grid, dim3(256), 0, s, q);
  } else {
    dim3 grid(groups, p.kv * kblocks * cblocks, 1);
    hipLaunchKernelGGL((wgrad_atomic_kernel<T>), grid, dim3(256), 0, s, p);
  }
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((wgrad_finalize_kernel<T>), dim3((unsigned)((f.total / 4 + 255) / 256)), dim3(256), 0, s, f);
  return hipGetLastError();
}

// Fixed-order variant: the same units, a contiguous run per workgroup, partial sums stored into
// slots and added up in workgroup order.  `max_wgs` = workgroups the caller's slots allow.
int CUMM_CAT(wgrad_ordered_resident_, CUMM_NAME)(bool wide) {
  using T = CUMM_ELEM;
  static int resident_of[2][16] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  int &resident = resident_of[wide ? 1 : 0][dev & 15];
  if (resident == 0) {
    int cus = 0, per_cu = 0;
    hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess)
      e = wide ? hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, wgrad_units_kernel<T, 2, 2, 1, true>, 256, 0)
               : hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, wgrad_units_kernel<T, 1, 1, 2, true>, 256, 0);
    if (e != hipSuccess) return 0;
    resident = cus * per_cu > 0 ? cus * per_cu : 1;
  }
  return resident;
}

hipError_t CUMM_CAT(launch_wgrad_ordered_, CUMM_NAME)(const WgradParams &p, const WgradPrepareParams &pre,
                                                      const WgradOrderedParams &f, bool wide, int wgs, hipStream_t s) {
  using T = CUMM_ELEM;
  if (p.num_red == 0 || p.kv == 0 || wgs < 1) return hipSuccess;
  if (!(wide ? counted_waits_hold<wgrad_units_kernel<T, 2, 2, 1, true>>() : counted_waits_hold<wgrad_units_kernel<T, 1, 1, 2, true>>()))
    return hipErrorNotSupported;
  hipLaunchKernelGGL(wgrad_prepare_kernel, dim3(p.kv), dim3(256), 0, s, pre);   // lists only: no image to zero
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (wide) hipLaunchKernelGGL((wgrad_units_kernel<T, 2, 2, 1, true>), dim3(wgs), dim3(256), 0, s, p);
  else hipLaunchKernelGGL((wgrad_units_kernel<T, 1, 1, 2, true>), dim3(wgs), dim3(256), 0, s, p);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((wgrad_finalize_ordered_kernel<T>), dim3((unsigned)((f.total / 4 + 31) / 32)), dim3(256), 0, s, f);
  return hipGetLastError();
}
#endif

}  // namespace cummhip
