// Seeded random weights from a counter generator: element i of a tensor is a function of (key, i) alone, so a
// tensor can be drawn in any order, in pieces, on any device, and comes out the same (the host twin of this
// kernel is weights/random_init.py, held to it bit by bit by a test).
//   h_j = mix(key + (3 i + j) * 0x9E3779B97F4A7C15), j = 0, 1, 2      (the splitmix64 finaliser)
//   s   = the sum of the twelve 16-bit fields of h_0, h_1, h_2       (Irwin-Hall: mean 6 * 65535, deviation 65536)
//   x   = float(s - 393210) * scale (+ offset)                        one rounding each, never contracted
// which is normal to within 1% out to three deviations and bounded by six.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

__device__ __forceinline__ uint64_t mix64(uint64_t x) {
  x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 27; x *= 0x94D049BB133111EBull;
  x ^= x >> 31;
  return x;
}

__device__ __forceinline__ int fields16(uint64_t h) {
  return int(h & 0xFFFF) + int((h >> 16) & 0xFFFF) + int((h >> 32) & 0xFFFF) + int(h >> 48);
}

template <typename T>
__global__ __launch_bounds__(256) void random_fill_kernel(T* __restrict__ dst, int64_t n, uint64_t key, int64_t first,
                                                          float scale, float offset, int add_offset) {
  int64_t i = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t step = int64_t(gridDim.x) * blockDim.x;
  for (; i < n; i += step) {
    const uint64_t c = 3ull * uint64_t(first + i);
    const int s = fields16(mix64(key + c * 0x9E3779B97F4A7C15ull)) + fields16(mix64(key + (c + 1) * 0x9E3779B97F4A7C15ull)) +
                  fields16(mix64(key + (c + 2) * 0x9E3779B97F4A7C15ull));
    float x = __fmul_rn(float(s - 393210), scale);
    if (add_offset) x = __fadd_rn(x, offset);
    dst[i] = from_float<T>(x);
  }
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_random_fill(void* stream, int dtype, void* dst, int64_t n, uint64_t key, int64_t first, float scale,
                              float offset, int add_offset) {
  SP_REQUIRE(n >= 0 && first >= 0, "sp_random_fill: bad range");
  if (n == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int blocks = (int)((n + 255) / 256 > 16384 ? 16384 : (n + 255) / 256);
  if (dtype == kF32) random_fill_kernel<float><<<blocks, 256, 0, s>>>((float*)dst, n, key, first, scale, offset, add_offset);
  else if (dtype == kBF16) random_fill_kernel<bf16_t><<<blocks, 256, 0, s>>>((bf16_t*)dst, n, key, first, scale, offset, add_offset);
  else SP_REQUIRE(false, "sp_random_fill: unsupported dtype %d", dtype);
  return check_launch("sp_random_fill");
}
