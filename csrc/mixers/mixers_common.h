// Helpers shared by the sequence-mixer translation units (csrc/mixers/*.hip): loads / stores of
// activations that are float or bf16 (raw uint16_t), and the host-side dtype dispatch.
#pragma once

#include "common.h"

namespace xgm {
using xgk::bf2f;
using xgk::block_sum;
using xgk::f2bf;
using xgk::wave_max;
using xgk::wave_sum;
typedef uint16_t bf16;

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16>(const bf16* p) { return bf2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16>(bf16* p, float v) { *p = f2bf(v); }

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + expf(-x)); }

// 4 consecutive elements (16-byte / 8-byte aligned)
__device__ __forceinline__ void ld4(const float* p, float (&f)[4]) {
  const float4 v = *reinterpret_cast<const float4*>(p);
  f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
}
__device__ __forceinline__ void ld4(const bf16* p, float (&f)[4]) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  f[0] = __uint_as_float(v.x << 16), f[1] = __uint_as_float(v.x & 0xFFFF0000u);
  f[2] = __uint_as_float(v.y << 16), f[3] = __uint_as_float(v.y & 0xFFFF0000u);
}
__device__ __forceinline__ void st4(float* p, const float (&f)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
}
__device__ __forceinline__ void st4(bf16* p, const float (&f)[4]) {
  *reinterpret_cast<uint2*>(p) = make_uint2(xgk::pack2(f[0], f[1]), xgk::pack2(f[2], f[3]));
}

__device__ __forceinline__ float siluf(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplusf(float x) { return x > 20.f ? x : log1pf(expf(x)); }

}  // namespace xgm

#define XGM_DISPATCH_T(f32, ...)      \
  if (f32) {                          \
    using T = float;                  \
    __VA_ARGS__                       \
  } else {                            \
    using T = bf16;                   \
    __VA_ARGS__                       \
  }
