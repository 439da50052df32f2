// Instantiations of the LDS-tiled GEMM for one element type (selected with -DCUMM_ELEM=...).
#include "launch.h"

namespace cummhip {

#define CUMM_CAT_(a, b) a##b
#define CUMM_CAT(a, b) CUMM_CAT_(a, b)

template <class T, int BM, int BN>
static hipError_t launch_xy(bool xk, bool yk, const TileGemmParams &p, dim3 grid, hipStream_t s) {
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;
  if (xk && yk) hipLaunchKernelGGL((tilegemm_kernel<T, true, true, BM, BN, 1>), grid, dim3(256), 0, s, p);
  else if (xk && !yk) hipLaunchKernelGGL((tilegemm_kernel<T, true, false, BM, BN, 1>), grid, dim3(256), 0, s, p);
  else if (!xk && yk) hipLaunchKernelGGL((tilegemm_kernel<T, false, true, BM, BN, 1>), grid, dim3(256), 0, s, p);
  else hipLaunchKernelGGL((tilegemm_kernel<T, false, false, BM, BN, 1>), grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

hipError_t CUMM_CAT(launch_tilegemm_, CUMM_NAME)(int tm, int tn, bool xk, bool yk,
                                                 const TileGemmParams &p, dim3 grid, hipStream_t s) {
  using T = CUMM_ELEM;
  if (tm == 64 && tn == 64) return launch_xy<T, 2, 2>(xk, yk, p, grid, s);
  if (tm == 128 && tn == 128) return launch_xy<T, 4, 4>(xk, yk, p, grid, s);
  return hipErrorInvalidValue;
}

#ifndef CUMM_NO_WGRAD_ATOMIC
hipError_t CUMM_CAT(launch_wgrad_atomic_, CUMM_NAME)(const WgradParams &p, const WgradPrepareParams &pre,
                                                     const WgradFinalizeParams &f, hipStream_t s) {
  using T = CUMM_ELEM;
  const int groups = (p.num_red + p.tiles_per_wg - 1) / p.tiles_per_wg;
  const int kblocks = (p.K + 63) / 64, cblocks = (p.C + 63) / 64;
  if (groups == 0 || p.kv == 0) return hipSuccess;
  hipError_t e;
  if (p.live_list != nullptr) {
    // lists + zeroed image, then a resident grid that walks the units
    static int resident_of[16] = {};
    int dev = 0;
    e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    int &resident = resident_of[dev & 15];
    if (resident == 0) {
      int cus = 0, per_cu = 0;
      e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, wgrad_units_kernel<T>, 256, 0);
      if (e != hipSuccess) return e;
      resident = cus * per_cu > 0 ? cus * per_cu : 1;
    }
    hipLaunchKernelGGL(wgrad_prepare_kernel, dim3(p.kv + 256), dim3(256), 0, s, pre);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
    // never more workgroups than units can exist
    const long long max_units = ((long long)groups * p.kv + p.kv) * kblocks * cblocks;
    hipLaunchKernelGGL((wgrad_units_kernel<T>), dim3((unsigned)(max_units < resident ? max_units : resident)),
                       dim3(256), 0, s, p);
  } else {
    dim3 grid(groups, p.kv * kblocks * cblocks, 1);
    hipLaunchKernelGGL((wgrad_atomic_kernel<T>), grid, dim3(256), 0, s, p);
  }
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((wgrad_finalize_kernel<T>), dim3((unsigned)((f.total / 4 + 255) / 256)), dim3(256), 0, s, f);
  return hipGetLastError();
}
#endif

}  // namespace cummhip
