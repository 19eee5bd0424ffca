// Shared helpers of the HIP kernels: storage types, conversions, reductions, error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

namespace sprout {

// Element type codes of the C interface.
enum DType : int { kF32 = 0, kBF16 = 1 };

struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16_t v) { return __uint_as_float(uint32_t(v.bits) << 16); }

// Round to nearest even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) { return bf16_t{f32_to_bf16_bits(f)}; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result. `scratch` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, waves = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

// Error text of the last failed call on this thread.
void set_error(const char* fmt, ...);
int check_launch(const char* what);

}  // namespace sprout

#define SP_REQUIRE(cond, ...)                 \
  do {                                        \
    if (!(cond)) {                            \
      sprout::set_error(__VA_ARGS__);         \
      return 1;                               \
    }                                         \
  } while (0)
