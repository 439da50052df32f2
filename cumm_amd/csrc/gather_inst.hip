// Stand-alone row gather and row scatter-add (what the per-offset "native" path of the reference's
// callers uses around a plain GEMM; cumm/gemm/gather.py:127-256 GatherKernelV2 / Gather.gather,
// :259-389 ScatterKernel / Scatter.scatter):
//   gather:       output[i, :]           = input[indices[i], :]      i < m
//   scatter-add:  output[indices[i], :] += input[i, :]               i < m, indices unique
// Both are copies bound by HBM bandwidth: one lane moves 16 bytes (4 when rows are not multiples
// of 16 bytes or a pointer is not 16-byte aligned), consecutive lanes take consecutive pieces of a
// row, then the next row, so that every access of a wave covers whole rows; there is one piece
// per lane and enough waves per CU (8 per SIMD) to keep the memory pipeline full without
// unrolling.  An index outside the source (gather) reads zeros; a row whose index is outside the
// destination (scatter-add) is dropped.
#include <hip/hip_runtime.h>

#include "launch.h"

namespace cummhip {

namespace {

template <class V>
__global__ __launch_bounds__(256) void gather_rows_kernel(const RowMoveParams p) {
  const uint64_t t = blockIdx.x * 256ull + threadIdx.x;
  if (t >= p.pieces) return;
  const uint64_t row = p.shift >= 0 ? t >> p.shift : t / p.per_row;
  const uint64_t piece = t - row * p.per_row;
  const int32_t src = p.indices[row];
  V v = {};
  if (src >= 0 && src < p.rows_other) v = reinterpret_cast<const V *>(p.src)[(uint64_t)src * p.per_row + piece];
  reinterpret_cast<V *>(p.dst)[t] = v;
}

template <class T> struct AddWords;
template <> struct AddWords<float> {
  static __device__ __forceinline__ uint32_t add(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b));
  }
};
// two 16-bit elements per word: each sum is formed in fp32 and rounded once to the element type
template <class T> struct AddWords {
  static __device__ __forceinline__ uint32_t add(uint32_t a, uint32_t b) {
    using E = Elem<T>;
    const uint16_t lo = E::from_float(E::to_float((uint16_t)a) + E::to_float((uint16_t)b));
    const uint16_t hi = E::from_float(E::to_float((uint16_t)(a >> 16)) + E::to_float((uint16_t)(b >> 16)));
    return (uint32_t)lo | ((uint32_t)hi << 16);
  }
};

template <int W> struct Words;   // W 32-bit words moved by one lane
template <> struct Words<1> { typedef uint32_t type; };
template <> struct Words<4> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

template <class T, int W>
__global__ __launch_bounds__(256) void scatter_add_rows_kernel(const RowMoveParams p) {
  typedef typename Words<W>::type V;
  const uint64_t t = blockIdx.x * 256ull + threadIdx.x;
  if (t >= p.pieces) return;
  const uint64_t row = p.shift >= 0 ? t >> p.shift : t / p.per_row;
  const uint64_t piece = t - row * p.per_row;
  const int32_t dst = p.indices[row];
  if (dst < 0 || dst >= p.rows_other) return;
  V *out = reinterpret_cast<V *>(p.dst) + ((uint64_t)dst * p.per_row + piece);
  const V a = reinterpret_cast<const V *>(p.src)[t];
  const V b = *out;
  V c;
  if constexpr (W == 1) {
    c = AddWords<T>::add(a, b);
  } else {
#pragma unroll
    for (int w = 0; w < W; ++w) c[w] = AddWords<T>::add(a[w], b[w]);
  }
  *out = c;
}

template <class K>
hipError_t launch_pieces(K kernel, const RowMoveParams &p, hipStream_t s) {
  if (p.pieces == 0) return hipSuccess;
  const uint64_t wgs = (p.pieces + 255ull) / 256ull;
  if (wgs > 0x7fffffffull) return hipErrorInvalidValue;
  hipLaunchKernelGGL(kernel, dim3((unsigned)wgs), dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gather_rows(const RowMoveParams &p, bool wide, hipStream_t s) {
  typedef uint32_t v4u __attribute__((ext_vector_type(4)));
  if (wide) return launch_pieces(gather_rows_kernel<v4u>, p, s);
  return launch_pieces(gather_rows_kernel<uint32_t>, p, s);
}

hipError_t launch_scatter_add_rows(const RowMoveParams &p, int dtype, bool wide, hipStream_t s) {
  switch (dtype) {
  case 0: return wide ? launch_pieces(scatter_add_rows_kernel<float, 4>, p, s) : launch_pieces(scatter_add_rows_kernel<float, 1>, p, s);
  case 7: return wide ? launch_pieces(scatter_add_rows_kernel<F16, 4>, p, s) : launch_pieces(scatter_add_rows_kernel<F16, 1>, p, s);
  case 12: return wide ? launch_pieces(scatter_add_rows_kernel<BF16, 4>, p, s) : launch_pieces(scatter_add_rows_kernel<BF16, 1>, p, s);
  default: return hipErrorInvalidValue;
  }
}

}  // namespace cummhip
