// Greedy and temperature sampling over float32 logits, two stages per row.
// Greedy: lowest index among the maxima; a row with a non-finite logit yields -1
// (reference: argmaxKernel, native/cuda-device.inc:97-115).
// Temperature: argmax of logits / temperature + Gumbel noise.  The noise of a column comes from a
// counter generator keyed by (seed, counter, column) only, so a request's draw does not depend on
// what else is in the batch or on the row it lands in.
#include <mutex>

#include "common.h"
#include "sprout_hip.h"

namespace sprout {

constexpr int SAMPLE_CHUNK = 2048;  // logits per first-stage block: two groups of four per thread

__device__ __forceinline__ uint64_t mix64(uint64_t z) {  // splitmix64 finaliser
  z += 0x9e3779b97f4a7c15ull;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float gumbel(uint64_t seed, uint32_t counter, uint32_t column) {
  const uint64_t h = mix64(mix64(seed ^ (uint64_t(counter) << 32)) + column);
  const float u = (float(uint32_t(h >> 40)) + 0.5f) * (1.0f / 16777216.0f);  // (0, 1)
  return -logf(-logf(u));
}

__device__ __forceinline__ void take_better(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

__global__ __launch_bounds__(256) void sample_stage1(const float* __restrict__ logits,
                                                     const float* __restrict__ temperature,
                                                     const int64_t* __restrict__ seed,
                                                     const int32_t* __restrict__ counter,
                                                     float* __restrict__ part_value, int* __restrict__ part_index,
                                                     int V, int chunks) {
  __shared__ float sv[4];
  __shared__ int si[4];
  __shared__ int sbad[4];
  const int r = blockIdx.y, chunk = blockIdx.x;
  const float* row = logits + size_t(r) * V;
  const float temp = temperature ? temperature[r] : 0.f;
  const float inv_temp = temp > 0.f ? 1.0f / temp : 1.0f;
  const uint64_t sd = seed ? uint64_t(seed[r]) : 0;
  const uint32_t ctr = counter ? uint32_t(counter[r]) : 0;
  float bv = -INFINITY;
  int bi = 0x7fffffff, bad = 0;
  const int begin = chunk * SAMPLE_CHUNK, end = min(V, begin + SAMPLE_CHUNK);
  auto take = [&](float v, int i) {
    if (!isfinite(v)) bad = 1;
    if (temp > 0.f) v = v * inv_temp + gumbel(sd, ctr, uint32_t(i));
    take_better(bv, bi, v, i);
  };
  if ((V & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    // the row starts at a multiple of 16 bytes: both groups of four are requested before either is looked at
    float4 v[SAMPLE_CHUNK / 1024];
#pragma unroll
    for (int j = 0; j < SAMPLE_CHUNK / 1024; ++j) {
      const int i = begin + 4 * (int(threadIdx.x) + 256 * j);
      v[j] = i < end ? *reinterpret_cast<const float4*>(row + i) : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
#pragma unroll
    for (int j = 0; j < SAMPLE_CHUNK / 1024; ++j) {
      const int i = begin + 4 * (int(threadIdx.x) + 256 * j);
      if (i < end) { take(v[j].x, i); take(v[j].y, i + 1); take(v[j].z, i + 2); take(v[j].w, i + 3); }
    }
  } else {
    for (int i = begin + threadIdx.x; i < end; i += 256) take(row[i], i);
  }
  // within the wave by lane exchange, between the four waves through LDS
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    bad |= __shfl_xor(bad, o, 64);
    take_better(bv, bi, ov, oi);
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { sv[wave] = bv; si[wave] = bi; sbad[wave] = bad; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      sbad[0] |= sbad[w];
      take_better(sv[0], si[0], sv[w], si[w]);
    }
  }
  if (threadIdx.x == 0) {
    part_value[size_t(r) * chunks + chunk] = sv[0];
    part_index[size_t(r) * chunks + chunk] = sbad[0] ? -1 : si[0];
  }
}

__global__ __launch_bounds__(64) void sample_stage2(const float* __restrict__ part_value,
                                                    const int* __restrict__ part_index, int32_t* __restrict__ out,
                                                    int chunks) {
  const int r = blockIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff, bad = 0;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const int i = part_index[size_t(r) * chunks + c];
    if (i < 0) bad = 1;
    else take_better(bv, bi, part_value[size_t(r) * chunks + c], i);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int oi = __shfl_xor(bi, o, 64);
    bad |= __shfl_xor(bad, o, 64);
    take_better(bv, bi, ov, oi);
  }
  if (threadIdx.x == 0) out[r] = (bad || bi == 0x7fffffff) ? -1 : bi;
}

// The partial results of sp_sample_static: one copy of this array on every GPU that the library runs on, held
// until the process ends.  In host code the name `scratch` is only a handle for hipGetSymbolAddress; the
// address that kernels and copies take is the one that call returns, per device.
constexpr int kStaticScratchFloats = 64 * 1024;   // 256 KiB
static __device__ __align__(256) float scratch[kStaticScratchFloats];

constexpr int kMaxDevices = 64;
static float* g_scratch_of[kMaxDevices];   // device -> address of that device's copy of `scratch` (null: not asked yet)
static std::mutex g_scratch_lock;

// The current device's copy of `scratch`.  The first call on a device asks the runtime for its address.
static int static_scratch(float** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    set_error("sp_sample_static: no current device: %s", hipGetErrorString(e));
    return 1;
  }
  if (device < 0 || device >= kMaxDevices) {
    set_error("sp_sample_static: device %d is outside the %d devices the library keeps scratch for", device, kMaxDevices);
    return 1;
  }
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_of[device]) {
    void* address = nullptr;
    e = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !address) {
      set_error("sp_sample_static: cannot find the scratch array on device %d: %s", device, hipGetErrorString(e));
      return 1;
    }
    g_scratch_of[device] = static_cast<float*>(address);
  }
  *ptr = g_scratch_of[device];
  return 0;
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_sample_workspace_floats(int R, int V) {
  const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  return R * chunks * 2;
}

extern "C" int sp_sample(void* stream, const float* logits, const float* temperature, const int64_t* seed,
                         const int32_t* counter, int32_t* out, float* workspace, int R, int V) {
  SP_REQUIRE(R >= 0 && V > 0, "sp_sample: bad sizes R=%d V=%d", R, V);
  SP_REQUIRE(logits && out && workspace, "sp_sample: null argument");
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  float* part_value = workspace;
  int* part_index = (int*)(workspace + size_t(R) * chunks);
  sample_stage1<<<dim3(chunks, R), 256, 0, s>>>(logits, temperature, seed, counter, part_value, part_index, V, chunks);
  sample_stage2<<<R, 64, 0, s>>>(part_value, part_index, out, chunks);
  return check_launch("sp_sample");
}

extern "C" int sp_sample_static_max_floats() { return kStaticScratchFloats; }

// sp_sample with the partial results in the library's own device array: nothing is allocated.
extern "C" int sp_sample_static(void* stream, const float* logits, const float* temperature, const int64_t* seed,
                                const int32_t* counter, int32_t* out, int R, int V) {
  SP_REQUIRE(R >= 0 && V > 0, "sp_sample_static: bad sizes R=%d V=%d", R, V);
  SP_REQUIRE(logits && out, "sp_sample_static: null argument");
  if (R == 0) return 0;
  const int chunks = (V + SAMPLE_CHUNK - 1) / SAMPLE_CHUNK;
  const long long need = 2LL * R * chunks;
  SP_REQUIRE(need <= kStaticScratchFloats,
             "sp_sample_static: %d rows of %d logits need %lld floats of scratch, the static array holds %d "
             "(use sp_sample with a workspace of the caller's)", R, V, need, kStaticScratchFloats);
  float* ws = nullptr;
  if (static_scratch(&ws)) return 1;
  hipStream_t s = (hipStream_t)stream;
  // Every slot that the second stage reads is written by the first stage of the same call: nothing has to
  // start at zero, and what an earlier call left in the array is never read.
  float* part_value = ws;
  int* part_index = reinterpret_cast<int*>(ws + size_t(R) * chunks);
  sample_stage1<<<dim3(chunks, R), 256, 0, s>>>(logits, temperature, seed, counter, part_value, part_index, V, chunks);
  sample_stage2<<<R, 64, 0, s>>>(part_value, part_index, out, chunks);
  return check_launch("sp_sample_static");
}
