// Shared helpers of the liblvmix.so kernels (gfx950, 64-wide wavefronts).
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "lv_mixers.h"

namespace lvmix {

constexpr int kWave = 64;

// Activation element types: bf16 (stored as its 16 bits) or f32; all arithmetic is f32.
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const bf16_t* p) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(p->bits) << 16);
}
__device__ __forceinline__ void stf(float* p, float x) { *p = x; }
__device__ __forceinline__ void stf(bf16_t* p, float x) {
  __bf16 b = static_cast<__bf16>(x);   // round to nearest even (hardware conversion on gfx950)
  p->bits = __builtin_bit_cast(uint16_t, b);
}

// Four consecutive elements at once: 16-byte accesses of f32 rows, 8-byte accesses of bf16 rows (aligned by the caller).
__device__ __forceinline__ float4 ld4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
  const uint2 v = *reinterpret_cast<const uint2*>(p);
  return float4{__builtin_bit_cast(float, v.x << 16), __builtin_bit_cast(float, v.x & 0xffff0000u),
                __builtin_bit_cast(float, v.y << 16), __builtin_bit_cast(float, v.y & 0xffff0000u)};
}
__device__ __forceinline__ void st4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
  bf16_t a, b, c, d;
  stf(&a, v.x); stf(&b, v.y); stf(&c, v.z); stf(&d, v.w);
  *reinterpret_cast<uint2*>(p) = uint2{static_cast<uint32_t>(a.bits) | (static_cast<uint32_t>(b.bits) << 16),
                                       static_cast<uint32_t>(c.bits) | (static_cast<uint32_t>(d.bits) << 16)};
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, kWave);
  return x;
}
__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) x = fmaxf(x, __shfl_xor(x, o, kWave));
  return x;
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float siluf_(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplusf_(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

int fail(int code, const char* fmt, ...);
inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
int launched(const char* what);

}  // namespace lvmix
