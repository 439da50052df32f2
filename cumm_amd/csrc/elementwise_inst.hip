// Row-wise helper kernels around the GEMM / sparse-convolution kernels: HBM-bound elementwise and
// reduction work that a caller of the convolution needs between launches.
//
//   finish_rows      out[r, c] = cvt(act(alpha * acc[r, c] + beta * bias[c])) from an fp32 image of
//                    the result (the per-offset "native" convolution accumulates in fp32 and
//                    rounds once, here)
//   relu_backward    dst = grad where the forward output was positive, else 0
//   column_sum       dst[c] = cvt(sum over rows of src[r, c]) in fp32, in a fixed order (the
//                    gradient of a bias): per-block partial sums, then a sum over blocks in
//                    block order, so the result is the same from run to run
//
// All three move 16-byte pieces (8 two-byte elements), consecutive lanes on consecutive pieces.
#include "launch.h"

namespace cummhip {

namespace {

template <class T>
__device__ __forceinline__ void unpack8(const v4i &v, float (&f)[8]) {
  const uint16_t *h = reinterpret_cast<const uint16_t *>(&v);
#pragma unroll
  for (int x = 0; x < 8; ++x) f[x] = Elem<T>::to_float(h[x]);
}
template <class T>
__device__ __forceinline__ v4i pack8(const float (&f)[8]) {
  v4i v;
  uint16_t *h = reinterpret_cast<uint16_t *>(&v);
#pragma unroll
  for (int x = 0; x < 8; ++x) h[x] = Elem<T>::from_float(f[x]);
  return v;
}

// one thread per 8 consecutive channels of one row
template <class T>
__global__ __launch_bounds__(256) void finish_rows_kernel(const FinishRowsParams p) {
  const int64_t vecs_per_row = p.channels / 8;
  const int64_t total = p.rows * vecs_per_row;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / vecs_per_row;
    const int c = (int)(i - r * vecs_per_row) * 8;
    const v4f *ap = reinterpret_cast<const v4f *>(p.acc + r * p.channels + c);
    const v4f a0 = ap[0], a1 = ap[1];
    float b[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (p.bias != nullptr && p.beta != 0.0f)
      unpack8<T>(*reinterpret_cast<const v4i *>(reinterpret_cast<const uint16_t *>(p.bias) + c), b);
    float t[8];
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      const float a = x < 4 ? a0[x & 3] : a1[x & 3];
      // the fused form of the GEMM kernels' epilogue
      const float v = p.bias != nullptr && p.beta != 0.0f ? __builtin_fmaf(p.alpha, a, p.beta * b[x]) : p.alpha * a;
      t[x] = apply_act(v, p.act, p.act_alpha);
    }
    *reinterpret_cast<v4i *>(reinterpret_cast<uint16_t *>(p.out) + r * p.channels + c) = pack8<T>(t);
  }
}

template <class T>
__global__ __launch_bounds__(256) void relu_backward_kernel(v4i *dst, const v4i *grad, const v4i *out, size_t vecs) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < vecs; i += (size_t)gridDim.x * 256) {
    const v4i g = grad[i], o = out[i];
    const uint16_t *gh = reinterpret_cast<const uint16_t *>(&g);
    const uint16_t *oh = reinterpret_cast<const uint16_t *>(&o);
    v4i r;
    uint16_t *rh = reinterpret_cast<uint16_t *>(&r);
#pragma unroll
    for (int x = 0; x < 8; ++x) rh[x] = Elem<T>::to_float(oh[x]) > 0.0f ? gh[x] : (uint16_t)0;
    dst[i] = r;
  }
}

// partial[b][c] = sum of src[r][c] over the rows of block b.  Thread t takes the 8-channel piece
// t % V of the rows t / V, t / V + R, ... of its block (V pieces per row, R = 256 / V rows at a
// time); the R row lanes of a piece are then summed through LDS in lane order.
template <class T>
__global__ __launch_bounds__(256) void column_partial_kernel(const ColumnSumParams p) {
  __shared__ float lds[256][9];
  const int V = p.channels / 8;
  const int R = 256 / V;
  const int t = threadIdx.x;
  const int piece = t % V, lane_row = t / V;
  float s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (lane_row < R) {
    const int64_t r0 = (int64_t)blockIdx.x * p.rows_per_block;
    int64_t r1 = r0 + p.rows_per_block;
    if (r1 > p.rows) r1 = p.rows;
    for (int64_t r = r0 + lane_row; r < r1; r += R) {
      float f[8];
      unpack8<T>(*reinterpret_cast<const v4i *>(reinterpret_cast<const uint16_t *>(p.src) + r * p.channels + piece * 8), f);
#pragma unroll
      for (int x = 0; x < 8; ++x) s[x] += f[x];
    }
  }
#pragma unroll
  for (int x = 0; x < 8; ++x) lds[t][x] = s[x];
  __syncthreads();
  if (lane_row == 0) {
    for (int j = 1; j < R; ++j)
#pragma unroll
      for (int x = 0; x < 8; ++x) s[x] += lds[j * V + piece][x];
    float *dst = p.partial + (int64_t)blockIdx.x * p.channels + piece * 8;
#pragma unroll
    for (int x = 0; x < 8; ++x) dst[x] = s[x];
  }
}

// dst[c] = cvt(sum over blocks) in a fixed shape: sixteen threads per channel, thread j adds the j-th
// sixteenth of the blocks in block order (eight loads in flight at a time: one thread walking all
// 1024 blocks took 54 us), then the sixteen sums are added in order
template <class T>
__global__ __launch_bounds__(256) void column_final_kernel(const ColumnSumParams p) {
  __shared__ float part[16][17];
  const int cl = threadIdx.x & 15, j = threadIdx.x >> 4;
  const int c = blockIdx.x * 16 + cl;
  const int share = (p.blocks + 15) >> 4;
  const int b0 = j * share, b1 = b0 + share < p.blocks ? b0 + share : p.blocks;
  float s = 0.0f;
  if (c < p.channels) {
    for (int b = b0; b < b1; b += 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = b + u < b1 ? p.partial[(int64_t)(b + u) * p.channels + c] : 0.0f;
#pragma unroll
      for (int u = 0; u < 8; ++u) s += v[u];
    }
  }
  part[j][cl] = s;
  __syncthreads();
  if (j == 0 && c < p.channels) {
    float total = part[0][cl];
#pragma unroll
    for (int k = 1; k < 16; ++k) total += part[k][cl];
    reinterpret_cast<uint16_t *>(p.dst)[c] = Elem<T>::from_float(total);
  }
}

unsigned grid_for(size_t items) {
  size_t blocks = (items + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  return (unsigned)(blocks > 0 ? blocks : 1);
}

}  // namespace

hipError_t launch_finish_rows(const FinishRowsParams &p, bool bf16, hipStream_t s) {
  const size_t items = (size_t)p.rows * (size_t)(p.channels / 8);
  if (items == 0) return hipSuccess;
  if (bf16) hipLaunchKernelGGL(finish_rows_kernel<BF16>, dim3(grid_for(items)), dim3(256), 0, s, p);
  else hipLaunchKernelGGL(finish_rows_kernel<F16>, dim3(grid_for(items)), dim3(256), 0, s, p);
  return hipGetLastError();
}

hipError_t launch_relu_backward(void *dst, const void *grad, const void *out, size_t vecs, bool bf16, hipStream_t s) {
  if (vecs == 0) return hipSuccess;
  if (bf16)
    hipLaunchKernelGGL(relu_backward_kernel<BF16>, dim3(grid_for(vecs)), dim3(256), 0, s, reinterpret_cast<v4i *>(dst),
                       reinterpret_cast<const v4i *>(grad), reinterpret_cast<const v4i *>(out), vecs);
  else
    hipLaunchKernelGGL(relu_backward_kernel<F16>, dim3(grid_for(vecs)), dim3(256), 0, s, reinterpret_cast<v4i *>(dst),
                       reinterpret_cast<const v4i *>(grad), reinterpret_cast<const v4i *>(out), vecs);
  return hipGetLastError();
}

int column_sum_blocks(int64_t rows, int channels) {
  const int V = channels / 8;
  const int R = V > 0 && V <= 256 ? 256 / V : 1;
  // about 16 row steps per block, at most 1024 blocks
  int64_t blocks = (rows + (int64_t)R * 16 - 1) / ((int64_t)R * 16);
  if (blocks > 1024) blocks = 1024;
  return (int)(blocks > 0 ? blocks : 1);
}

hipError_t launch_column_sum(ColumnSumParams p, bool bf16, hipStream_t s) {
  p.blocks = column_sum_blocks(p.rows, p.channels);
  p.rows_per_block = (p.rows + p.blocks - 1) / p.blocks;
  if (bf16) {
    hipLaunchKernelGGL(column_partial_kernel<BF16>, dim3(p.blocks), dim3(256), 0, s, p);
    hipLaunchKernelGGL(column_final_kernel<BF16>, dim3((p.channels + 15) / 16), dim3(256), 0, s, p);
  } else {
    hipLaunchKernelGGL(column_partial_kernel<F16>, dim3(p.blocks), dim3(256), 0, s, p);
    hipLaunchKernelGGL(column_final_kernel<F16>, dim3((p.channels + 15) / 16), dim3(256), 0, s, p);
  }
  return hipGetLastError();
}

}  // namespace cummhip
