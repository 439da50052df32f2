// Host-side launch tables: one function per element type, defined in its own translation unit so
// that the kernel instantiations compile in parallel.
#pragma once
#include "rowgemm.h"
#include "tilegemm.h"
#include "wgrad_atomic.h"

namespace cummhip {

// returns hipSuccess, or hipErrorInvalidValue when no instantiation matches
hipError_t launch_rowgemm_f16(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);
hipError_t launch_rowgemm_bf16(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);
hipError_t launch_rowgemm_s8(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s);

hipError_t launch_tilegemm_f16(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                               hipStream_t s);
hipError_t launch_tilegemm_bf16(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                                hipStream_t s);
hipError_t launch_tilegemm_s8(int tm, int tn, bool xk, bool yk, const TileGemmParams &p, dim3 grid,
                              hipStream_t s);

// balanced backward-weight with fp32 atomics: main kernel then finalize (f16 / bf16 only)
hipError_t launch_wgrad_atomic_f16(const WgradParams &p, const WgradPrepareParams &pre, const WgradFinalizeParams &f, hipStream_t s);
hipError_t launch_wgrad_atomic_bf16(const WgradParams &p, const WgradPrepareParams &pre, const WgradFinalizeParams &f, hipStream_t s);

// tile shapes the tables above hold
inline bool rowgemm_has_tile(int tm, int tn) {
  return (tm == 64 || tm == 128) && (tn == 64 || tn == 128);
}
inline bool tilegemm_has_tile(int tm, int tn) {
  return (tm == 64 && tn == 64) || (tm == 128 && tn == 128);
}

}  // namespace cummhip
