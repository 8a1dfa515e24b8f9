// 16-bit pack / unpack and the SiLU-multiply arithmetic shared by the elementwise kernels and by the rank-r pass that
// takes SiLU(gate) * up as its input (internal).
#pragma once
#include "lf_common.h"

template <typename T> __device__ __forceinline__ void unpack8(const lf_u32x4& v, float f[8]);
template <> __device__ __forceinline__ void unpack8<__bf16>(const lf_u32x4& v, float f[8]) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t u = v[i];
    f[2 * i] = __builtin_bit_cast(float, u << 16);
    f[2 * i + 1] = __builtin_bit_cast(float, u & 0xffff0000u);
  }
}
template <> __device__ __forceinline__ void unpack8<_Float16>(const lf_u32x4& v, float f[8]) {
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const uint32_t u = v[i];  // a copy: bit_cast applied to the vector element itself reads element 0 for every i
    const v2 h = __builtin_bit_cast(v2, u);
    f[2 * i] = (float)h[0];
    f[2 * i + 1] = (float)h[1];
  }
}

template <typename T> __device__ __forceinline__ lf_u32x4 pack8(const float f[8]) {
  typedef T v2 __attribute__((ext_vector_type(2)));
  lf_u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const v2 h = {(T)f[2 * i], (T)f[2 * i + 1]};
    o[i] = __builtin_bit_cast(uint32_t, h);
  }
  return o;
}

template <typename T> __device__ __forceinline__ float round16(float v) { return (float)(T)v; }

// exp and reciprocal to one unit in the last place of fp32 each (the results are rounded to 16 bits)
__device__ __forceinline__ float sigmoid_f32(float a) { return __builtin_amdgcn_rcpf(1.0f + __expf(-a)); }

// eight elements of round16(round16(silu(a)) * b)
template <typename T> __device__ __forceinline__ lf_u32x4 silu_mul8(const lf_u32x4& a, const lf_u32x4& b) {
  float fa[8], fb[8];
  unpack8<T>(a, fa);
  unpack8<T>(b, fb);
#pragma unroll
  for (int e = 0; e < 8; e++) fa[e] = round16<T>(fa[e] * sigmoid_f32(fa[e])) * fb[e];
  return pack8<T>(fa);
}
