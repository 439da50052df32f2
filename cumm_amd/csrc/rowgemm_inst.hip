// Instantiations of the gather-rows GEMM for one element type (selected with -DCUMM_ELEM=...).
#include "launch.h"
#include "rowgemm_pipe.h"
#include "rowgemm_lds.h"
#include "rowgemm_wave.h"

namespace cummhip {

#ifndef CUMM_DW
#define CUMM_DW 1   // steps of weight slices in flight
#endif

#define CUMM_CAT_(a, b) a##b
#define CUMM_CAT(a, b) CUMM_CAT_(a, b)

// -DCUMM_WIDE=1 builds the same table with four-byte outputs (s32 / f32) under the name
// launch_rowgemm_wide_<type>, in a translation unit of its own
#ifndef CUMM_WIDE
#define CUMM_WIDE 0
#endif
constexpr bool kWide = CUMM_WIDE != 0;
#if CUMM_WIDE
#define CUMM_LAUNCH_NAME CUMM_CAT(launch_rowgemm_wide_, CUMM_NAME)
#else
#define CUMM_LAUNCH_NAME CUMM_CAT(launch_rowgemm_, CUMM_NAME)
#endif

// kernel offsets per batch of the chunked kernel: bounded by the two LDS stages (TN * 64 * KS
// bytes per offset and stage, at most 32 KB per workgroup) and by the registers that hold the
// batch's gathered rows
constexpr int batch_size(int RB, int TN, int KS) {
  int b = 4;
  while (b > 1 && (2 * b * TN * 64 * KS > 32768 || RB * KS * b > 16)) b >>= 1;
  return b;
}
// offsets per step of the pipelined kernel: two where both LDS stages then fit 32 KB
constexpr int step_width(int TN, int KS) { return 2 * 2 * TN * 64 * KS <= 32768 ? 2 : 1; }
// steps of gathered rows kept in flight: as many as fit about 48 registers
constexpr int rows_ahead(int RB, int KS, int BW) {
  int d = 2;
  while (d > 1 && (d + 1) * BW * RB * KS * 4 > 64) --d;
  return d;
}

// ring stages of the LDS-streaming kernel: three where they fit 64 KB, else two, else none
constexpr int lds_stages(int TM, int TN, int KS) {
  const int stage = (TM + TN) * KS * 64;
#ifdef CUMM_LDS_NS
  if (CUMM_LDS_NS * stage <= 65536) return CUMM_LDS_NS;
#endif
  return 3 * stage <= 65536 ? 3 : (2 * stage <= 65536 ? 2 : 0);
}

// tile shapes and element types that have a kernel for several mask words per position
template <class T, int TM, int TN>
constexpr bool has_mask_words_kernel() { return Elem<T>::kBytes == 2 && !kWide && TM == TN; }

template <class T, int NW, int RB, int TN, int KS, bool WT>
static hipError_t launch_one(const RowGemmParams &p, hipStream_t s) {
  constexpr int TM = NW * RB * 16;
  dim3 grid((p.n_pos + TM - 1) / TM, (p.k_out + TN - 1) / TN, 1);
  if (grid.x == 0 || grid.y == 0) return hipSuccess;
  constexpr int chunk_e = 4 * KS * Elem<T>::kPerVec;
  if (p.mask_words > 1) {
    // kernel volumes above 32 (the reference's dynamic-mask kernels): the LDS-streaming kernel
    // with up to four mask words per position, whole contraction or chunked
    if constexpr (has_mask_words_kernel<T, TM, TN>()) {
      if (WT ? p.w_stride_n != 1 : p.w_stride_c != 1) return hipErrorInvalidValue;
      constexpr int KSM = KS == 4 ? 2 : KS;
      constexpr int NSM = lds_stages(TM, TN, KSM);
      if constexpr (NSM > 0) {
        constexpr int chunk_m = 4 * KSM * Elem<T>::kPerVec;
        RowGemmParams q = p;
        const int nch = (p.c_in + chunk_m - 1) / chunk_m;
        while ((1 << q.chunk_shift) < nch) ++q.chunk_shift;
        if (q.chunk_shift <= 3 && counted_waits_hold<rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, KSM, NSM, WT, false, 4>>()) {
          hipLaunchKernelGGL((rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, KSM, NSM, WT, false, 4>), grid, dim3(256), 0, s, q);
          return hipGetLastError();
        }
      }
    }
    return hipErrorInvalidValue;
  }
  // A contraction longer than 128 bytes: the LDS-streaming kernel walking the contraction in
  // chunks of one stage row, rather than 256-byte rows with two stages or the register-gather
  // kernels.  Stage rows of 128 bytes; for the 128 x 128 tile, whose 128-byte stages are 32 KB
  // (two stages, two workgroups per CU), also rows of 64 bytes when the descriptor asks for three
  // stages: 16 KB each, three workgroups per CU, half as much again in flight per CU.  Launches
  // whose tiles have few kernel offsets are bound by the latency of their round trips and gain
  // (C = K = 128 bf16 at 1 M voxels, 2 pairs per voxel: forward 0.229 -> 0.220 ms, backward-input
  // 0.218 -> 0.194 ms, stride-2 128 -> 256 forward 0.838 -> 0.751 ms; four stages at two
  // workgroups per CU: no gain); tiles with many offsets are bound by their steps, and twice the
  // steps per offset cost them (125 offsets, C = K = 128: 0.239 -> 0.300 ms), as they do the
  // smaller tiles (64 x 128 at 1 M voxels: 0.258 -> 0.281 ms).
  if constexpr (KS == 4) {
    if constexpr (TM == 128 && TN == 128 && lds_stages(TM, TN, 1) == 3 && (!WT || Elem<T>::kBytes == 2)) {
      constexpr int chunk1 = 4 * 1 * Elem<T>::kPerVec;
      const int nch = (p.c_in + chunk1 - 1) / chunk1;
      int shift = 0;
      while ((1 << shift) < nch) ++shift;
      if (p.small_stages && shift <= 3 && (WT ? p.w_stride_n == 1 : p.w_stride_c == 1)) {
        if (counted_waits_hold<rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, 1, 3, WT, kWide>>()) {
          RowGemmParams q = p;
          q.chunk_shift = shift;
          hipLaunchKernelGGL((rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, 1, 3, WT, kWide>), grid, dim3(256), 0, s, q);
          return hipGetLastError();
        }
      }
    }
    constexpr int NS2 = lds_stages(TM, TN, 2);
    if constexpr (NS2 > 0 && (!WT || Elem<T>::kBytes == 2)) {
      constexpr int chunk2 = 4 * 2 * Elem<T>::kPerVec;
      const int nch = (p.c_in + chunk2 - 1) / chunk2;
      int shift = 0;
      while ((1 << shift) < nch) ++shift;
      if (shift <= 3 && (WT ? p.w_stride_n == 1 : p.w_stride_c == 1)) {
        if (counted_waits_hold<rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, 2, NS2, WT, kWide>>()) {
          RowGemmParams q = p;
          q.chunk_shift = shift;
          hipLaunchKernelGGL((rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, 2, NS2, WT, kWide>), grid, dim3(256), 0, s, q);
          return hipGetLastError();
        }
      }
    }
  }
  constexpr int NS = lds_stages(TM, TN, KS);
  if constexpr (NS > 0 && (!WT || Elem<T>::kBytes == 2)) {
    // the LDS-streaming kernel: 2 x 2 waves, each TM/2 rows by TN/2 channels
    if (p.c_in <= chunk_e && (WT ? p.w_stride_n == 1 : p.w_stride_c == 1)) {
      if constexpr (TM == 64 && TN == 64 && Elem<T>::kBytes == 2 && KS <= 2 && !kWide) {
        if (p.hint_slot != nullptr && grid.y == 1 && p.chunk_shift == 0 && p.mask != nullptr &&
            counted_waits_hold<rowgemm_lds_mixed_kernel<T, KS, WT>>()) {
          const dim3 with_spare(grid.x + (unsigned)mixed_spare_tiles((int)grid.x), 1, 1);
          hipLaunchKernelGGL((rowgemm_lds_mixed_kernel<T, KS, WT>), with_spare, dim3(256), 0, s, p);
          return hipGetLastError();
        }
      }
      if (counted_waits_hold<rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, KS, NS, WT, kWide>>()) {
        hipLaunchKernelGGL((rowgemm_lds_kernel<T, 2, 2, TM / 32, TN / 32, KS, NS, WT, kWide>), grid, dim3(256), 0, s, p);
        return hipGetLastError();
      }
    }
  }
  if (p.c_in <= chunk_e) {
    constexpr int BW = step_width(TN, KS);
    constexpr int DA = rows_ahead(RB, KS, BW);
    hipLaunchKernelGGL((rowgemm_pipe_kernel<T, NW, RB, TN, KS, WT, BW, DA, DA, CUMM_DW, kWide>), grid, dim3(NW * 64), 0, s, p);
  } else {
    if constexpr (KS == 4) {
      constexpr int B = batch_size(RB, TN, KS);
      hipLaunchKernelGGL((rowgemm_kernel<T, NW, RB, TN, KS, WT, B, kWide>), grid, dim3(NW * 64), 0, s, p);
    } else {
      return hipErrorInvalidValue;  // a contraction longer than one chunk always selects KS == 4
    }
  }
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

// One weight matrix, no masks, a contraction of at most 128 two-byte elements: the kernel that keeps
// the matrix in registers (rowgemm_wave.h); the descriptor's tile shape then only names the launch.
template <class T, int KS, bool WT>
static hipError_t launch_wave(const RowGemmParams &p, hipStream_t s) {
  if constexpr (Elem<T>::kBytes == 2) {
    if (!counted_waits_hold<rowgemm_wave_kernel<T, KS, WT, kWide>>()) return hipErrorNotSupported;   // (the caller goes on)
    const int n_blocks = (p.n_pos + 15) / 16;
    if (n_blocks == 0 || p.k_out <= 0) return hipSuccess;
    static int resident_of[16] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    int &resident = resident_of[dev & 15];
    if (resident == 0) {
      int cus = 0, per_cu = 0;
      e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      if (e == hipSuccess) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, rowgemm_wave_kernel<T, KS, WT, kWide>, 256, 0);
      if (e != hipSuccess) return e;
      resident = cus * per_cu > 0 ? cus * per_cu : 1;
    }
    const int want = (n_blocks + 7) / 8;   // four waves, two row blocks per trip each
    dim3 grid((unsigned)(want < resident ? want : resident), (unsigned)((p.k_out + 63) / 64), 1);
    hipLaunchKernelGGL((rowgemm_wave_kernel<T, KS, WT, kWide>), grid, dim3(256), 0, s, p);
    return hipGetLastError();
  } else {
    return hipErrorInvalidValue;
  }
}

hipError_t CUMM_LAUNCH_NAME(int tm, int tn, int ks, bool wt, const RowGemmParams &p, hipStream_t s) {
  using T = CUMM_ELEM;
  if constexpr (Elem<T>::kBytes == 2) {
    // (up to 64 output channels: a second column block would gather the rows a second time)
    if (p.mask == nullptr && p.kv == 1 && p.gather_by_pos && p.c_in <= 32 * ks && p.k_out <= 64 &&
        (wt ? p.w_stride_n == 1 : p.w_stride_c == 1) && (tm == 64 || tm == 128) && (tn == 64 || tn == 128)) {
      hipError_t e = hipErrorNotSupported;
      switch (ks) {
      case 1: e = wt ? launch_wave<T, 1, true>(p, s) : launch_wave<T, 1, false>(p, s); break;
      case 2: e = wt ? launch_wave<T, 2, true>(p, s) : launch_wave<T, 2, false>(p, s); break;
      case 4: e = wt ? launch_wave<T, 4, true>(p, s) : launch_wave<T, 4, false>(p, s); break;
      }
      if (e != hipErrorNotSupported) return e;
    }
  }
  if (tm == 64 && tn == 64) return launch_ks<T, 4, 1, 64>(ks, wt, p, s);
  if (tm == 128 && tn == 64) return launch_ks<T, 4, 2, 64>(ks, wt, p, s);
  if (tm == 64 && tn == 128) return launch_ks<T, 4, 1, 128>(ks, wt, p, s);
  if (tm == 128 && tn == 128) return launch_ks<T, 4, 2, 128>(ks, wt, p, s);
  return hipErrorInvalidValue;
}

}  // namespace cummhip
