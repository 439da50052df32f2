// Instantiations of the gather-rows GEMM for one element type (selected with -DCUMM_ELEM=...).
#include "launch.h"

namespace cummhip {

#define CUMM_CAT_(a, b) a##b
#define CUMM_CAT(a, b) CUMM_CAT_(a, b)

template <class T, int NW, int RB, int TN, int KS, bool WT>
static hipError_t launch_one(const RowGemmParams &p, hipStream_t s) {
  constexpr int TM = NW * RB * 16;
  dim3 grid((p.n_pos + TM - 1) / TM, (p.k_out + TN - 1) / TN, 1);
  if (grid.x == 0 || grid.y == 0) return hipSuccess;
  hipLaunchKernelGGL((rowgemm_kernel<T, NW, RB, TN, KS, WT>), grid, dim3(NW * 64), 0, s, p);
  return hipGetLastError();
}

template <class T, int NW, int RB, int TN>
static hipError_t launch_ks(int ks, bool wt, const RowGemmParams &p, hipStream_t s) {
  if (!wt) {
    switch (ks) {
    case 1: return launch_one<T, NW, RB, TN, 1, false>(p, s);
    case 2: return launch_one<T, NW, RB, TN, 2, false>(p, s);
    case 4: return launch_one<T, NW, RB, TN, 4, false>(p, s);
    }
  } else {
    switch (ks) {
    case 1: return launch_one<T, NW, RB, TN, 1, true>(p, s);
    case 2: return launch_one<T, NW, RB, TN, 2, true>(p, s);
    case 4: return launch_one<T, NW, RB, TN, 4, true>(p, s);
    }
  }
  return hipErrorInvalidValue;
}

hipError_t CUMM_CAT(launch_rowgemm_, CUMM_NAME)(int tm, int tn, int ks, bool wt,
                                                const RowGemmParams &p, hipStream_t s) {
  using T = CUMM_ELEM;
  if (tm == 64 && tn == 64) return launch_ks<T, 4, 1, 64>(ks, wt, p, s);
  if (tm == 128 && tn == 64) return launch_ks<T, 4, 2, 64>(ks, wt, p, s);
  if (tm == 64 && tn == 128) return launch_ks<T, 4, 1, 128>(ks, wt, p, s);
  if (tm == 128 && tn == 128) return launch_ks<T, 4, 2, 128>(ks, wt, p, s);
  return hipErrorInvalidValue;
}

}  // namespace cummhip
