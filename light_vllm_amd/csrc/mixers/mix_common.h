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
