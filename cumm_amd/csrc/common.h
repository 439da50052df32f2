// Shared device/host helpers for the gfx950 kernels of libcummhip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace cummhip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// element tags ---------------------------------------------------------------
struct F16 {};
struct BF16 {};
struct S8 {};

template <class T> struct Elem;
template <> struct Elem<F16> {
  using Acc = float;
  using AccV = v4f;
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;   // elements in one 16-byte fragment
  static constexpr int kMfmaK = 32;   // contraction length of one 16x16 MFMA
  static __device__ __forceinline__ v4f mfma(v4i a, v4i b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a),
                                                  __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) {
    return (float)__builtin_bit_cast(_Float16, bits);
  }
  static __device__ __forceinline__ uint16_t from_float(float x) {
    return __builtin_bit_cast(uint16_t, (_Float16)x);  // v_cvt_f16_f32: round to nearest even
  }
};
template <> struct Elem<BF16> {
  using Acc = float;
  using AccV = v4f;
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  static constexpr int kMfmaK = 32;
  static __device__ __forceinline__ v4f mfma(v4i a, v4i b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a),
                                                   __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) {
    return __builtin_bit_cast(float, (uint32_t)bits << 16);
  }
  // round to nearest even on bit 16, NaN -> 0x7FFF
  // (bfloat16_t(float), include/tensorview/gemm/dtypes/bfloat16.h:86-111 of the reference)
  static __device__ __forceinline__ uint16_t from_float(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if (x != x) return 0x7FFF;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
  }
};
template <> struct Elem<S8> {
  using Acc = int;
  using AccV = v4i;
  static constexpr int kBytes = 1;
  static constexpr int kPerVec = 16;
  static constexpr int kMfmaK = 64;
  static __device__ __forceinline__ v4i mfma(v4i a, v4i b, v4i c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
};

// activations: UnaryActivation, cumm/gemm/gemmmath/__init__.py:181-214 of the reference
__device__ __forceinline__ float apply_act(float x, int act, float act_alpha) {
  switch (act) {
  case 1: return x > 0.0f ? x : 0.0f;
  case 2: return 1.0f / (1.0f + expf(-x));
  case 3: return x >= 0.0f ? x : x * act_alpha;
  default: return x;
  }
}

// float -> s8: clamp to [-128,127] then round half to even; NaN -> 0
// (Int8Inference clamp + cvt.rni.sat.s8.f32, cumm/gemm/output_op/linear.py:327-351,
//  include/tensorview/gemm/math/numeric_convert.h:171-192 of the reference)
// Three instructions: round half to even, convert (the hardware conversion saturates and turns
// NaN into 0; written as asm because the C cast is undefined out of range), clamp the integer.
// Clamping after the rounding equals clamping before it: the bounds are integers.
__device__ __forceinline__ int f32_to_s8(float t) {
  const float q = __builtin_rintf(t);
  int i;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(i) : "v"(q));
  i = i > 127 ? 127 : i;
  return i < -128 ? -128 : i;
}

// low bytes of four integers as one dword (three v_perm_b32)
__device__ __forceinline__ int pack4_bytes(int b0, int b1, int b2, int b3) {
  const uint32_t lo = __builtin_amdgcn_perm((uint32_t)b1, (uint32_t)b0, 0x0c0c0400u);
  const uint32_t hi = __builtin_amdgcn_perm((uint32_t)b3, (uint32_t)b2, 0x0c0c0400u);
  return (int)__builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

__device__ __forceinline__ uint32_t wave_or(uint32_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v |= (uint32_t)__shfl_xor((int)v, off, 64);
  return v;
}

}  // namespace cummhip
