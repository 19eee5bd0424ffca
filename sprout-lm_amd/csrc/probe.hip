// Two probes of the machine for the benchmark's report: what a kernel that only reads gets from memory, and
// what a kernel that only multiplies gets from the matrix cores.  Measured figures stand beside the published
// peaks; nothing in the engine depends on them.
#include "mfma.h"
#include "sprout_hip.h"

namespace sprout {

// Every thread reads 16 bytes at a time, 8 loads in flight, striding over the buffer with the whole grid.
__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ data, size_t vectors, float* __restrict__ sink) {
  const size_t stride = size_t(gridDim.x) * blockDim.x;
  uint32_t mix = 0;
  size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
  for (; i + 7 * stride < vectors; i += 8 * stride) {
    uint4 v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = data[i + j * stride];
#pragma unroll
    for (int j = 0; j < 8; ++j) mix ^= v[j].x ^ v[j].y ^ v[j].z ^ v[j].w;
  }
  for (; i < vectors; i += stride) {
    const uint4 v = data[i];
    mix ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (mix == 0x5eed5eedu) sink[0] = 1.f;     // keeps the loads; the value does not occur in the zeroed buffer
}

// Each wave keeps four independent chains of 32x32x16 bfloat16 products going: no memory, no dependencies
// between neighbouring instructions.
__global__ __launch_bounds__(256) void probe_mfma_kernel(int iterations, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<__bf16>(float(threadIdx.x % 7) * 0.125f);
    b[i] = static_cast<__bf16>(float(threadIdx.x % 5) * 0.25f);
  }
  floatx16 c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) c[j][i] = 0.f;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int j = 0; j < 4; ++j) c[j] = mfma32(a, b, c[j]);
  }
  float total = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) total += c[j][i];
  if (total == -1.f) sink[0] = total;
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_probe_read(void* stream, const void* data, int64_t bytes, int blocks, float* sink) {
  SP_REQUIRE(data && sink && bytes >= 16 && blocks > 0, "sp_probe_read: a buffer of at least 16 bytes, blocks and a sink are needed");
  probe_read_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(reinterpret_cast<const uint4*>(data), size_t(bytes) / 16, sink);
  return check_launch("sp_probe_read");
}

// Runs `blocks` blocks of four waves, `iterations` x 4 products of 32x32x16 each: returns through *flops what one
// launch computes (2 x 32 x 32 x 16 operations a product).
extern "C" int sp_probe_mfma(void* stream, int blocks, int iterations, float* sink, double* flops) {
  SP_REQUIRE(blocks > 0 && iterations > 0 && sink, "sp_probe_mfma: bad arguments");
  probe_mfma_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(iterations, sink);
  if (flops) *flops = double(blocks) * 4.0 * double(iterations) * 4.0 * 2.0 * 32.0 * 32.0 * 16.0;
  return check_launch("sp_probe_mfma");
}
