// out[T, N] = a[T, K] . w[N, K]^T (+ bias) with float32 products and sums, for any sizes and any
// mix of float32 / bfloat16 operands.  This is the exact path (no matrix-core instruction is used,
// so every product is a true float32 fma) and the fallback for operand mixes the MFMA kernels refuse.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

constexpr int GT = 64;   // tile of tokens and of output columns
constexpr int GK = 16;   // depth of one staging step

// Epilogue modes of the C interface.
enum { kStore = 0, kAccumulate = 1, kStoreF32 = 2 };

template <typename TA, typename TW, typename TB, typename TO, int MODE>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                           const TB* __restrict__ bias, TO* __restrict__ out,
                                                           int T, int N, int K) {
  __shared__ float As[GK][GT + 4];
  __shared__ float Ws[GK][GT + 4];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int t0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GK) {
    // 64 rows x 16 depth per operand; 256 threads load 4 elements each
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = threadIdx.x + i * 256;
      const int r = idx / GK, k = idx % GK;
      const bool kin = k0 + k < K;
      As[k][r] = (kin && t0 + r < T) ? to_float(a[size_t(t0 + r) * K + k0 + k]) : 0.f;
      Ws[k][r] = (kin && n0 + r < N) ? to_float(w[size_t(n0 + r) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = t0 + ty * 4 + i;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += to_float(bias[n]);
      const size_t o = size_t(t) * N + n;
      if (MODE == kAccumulate) out[o] = from_float<TO>(to_float(out[o]) + v);
      else out[o] = from_float<TO>(v);
    }
  }
}

// Few tokens: the weights are read once, at the speed of memory.  A wave owns two rows of w; its lanes
// share K four elements at a time and the sums meet by lane shuffles.  K must be a multiple of 4.
constexpr int RT = 16;   // most tokens of the row kernel

__device__ __forceinline__ void load4(const float* p, float v[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float v[4]) {
  const uint2 x = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
  v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
}

template <typename TA, typename TW, typename TB, typename TO, int MODE>
__global__ __launch_bounds__(256) void gemm_rows_kernel(const TA* __restrict__ a, const TW* __restrict__ w,
                                                        const TB* __restrict__ bias, TO* __restrict__ out,
                                                        int T, int N, int K) {
  const int lane = threadIdx.x & 63;
  const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * 2;
  if (n0 >= N) return;
  const int n1 = min(n0 + 1, N - 1);   // an odd N: the last wave reads its one row twice
  float acc[2][RT] = {};
#pragma unroll 2
  for (int k = lane * 4; k < K; k += 256) {
    float w0[4], w1[4];
    load4(w + size_t(n0) * K + k, w0);
    load4(w + size_t(n1) * K + k, w1);
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      if (t < T) {
        float av[4];
        load4(a + size_t(t) * K + k, av);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          acc[0][t] = fmaf(av[i], w0[i], acc[0][t]);
          acc[1][t] = fmaf(av[i], w1[i], acc[1][t]);
        }
      }
    }
  }
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (t >= T) break;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      float v = wave_sum(acc[r][t]);
      const int n = n0 + r;
      if (lane == 0 && n < N) {
        if (bias) v += to_float(bias[n]);
        const size_t o = size_t(t) * N + n;
        if (MODE == kAccumulate) out[o] = from_float<TO>(to_float(out[o]) + v);
        else out[o] = from_float<TO>(v);
      }
    }
  }
}

template <typename TA, typename TW, typename TB>
int launch_generic(hipStream_t s, const void* a, const void* w, const void* bias, int mode, int out_dtype,
                   void* out, int T, int N, int K) {
  dim3 grid((N + GT - 1) / GT, (T + GT - 1) / GT);
  const TA* ap = (const TA*)a;
  const TW* wp = (const TW*)w;
  const TB* bp = (const TB*)bias;
  if (T <= RT && K % 4 == 0 && (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) % 16 == 0) {
    const int blocks = (N + 7) / 8;
    if (mode == kAccumulate)
      gemm_rows_kernel<TA, TW, TB, float, kAccumulate><<<blocks, 256, 0, s>>>(ap, wp, bp, (float*)out, T, N, K);
    else if (mode == kStoreF32 || out_dtype == kF32)
      gemm_rows_kernel<TA, TW, TB, float, kStore><<<blocks, 256, 0, s>>>(ap, wp, bp, (float*)out, T, N, K);
    else
      gemm_rows_kernel<TA, TW, TB, bf16_t, kStore><<<blocks, 256, 0, s>>>(ap, wp, bp, (bf16_t*)out, T, N, K);
    return check_launch("sp_gemm (rows)");
  }
  if (mode == kAccumulate)
    gemm_generic_kernel<TA, TW, TB, float, kAccumulate><<<grid, 256, 0, s>>>(ap, wp, bp, (float*)out, T, N, K);
  else if (mode == kStoreF32 || out_dtype == kF32)
    gemm_generic_kernel<TA, TW, TB, float, kStore><<<grid, 256, 0, s>>>(ap, wp, bp, (float*)out, T, N, K);
  else
    gemm_generic_kernel<TA, TW, TB, bf16_t, kStore><<<grid, 256, 0, s>>>(ap, wp, bp, (bf16_t*)out, T, N, K);
  return check_launch("sp_gemm (generic)");
}

template <typename TA, typename TW>
int launch_generic_bias(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode,
                        int out_dtype, void* out, int T, int N, int K) {
  if (bias && bias_dtype == kBF16) return launch_generic<TA, TW, bf16_t>(s, a, w, bias, mode, out_dtype, out, T, N, K);
  return launch_generic<TA, TW, float>(s, a, w, bias, mode, out_dtype, out, T, N, K);
}

int gemm_generic(hipStream_t s, int a_dtype, const void* a, int w_dtype, const void* w, int bias_dtype,
                 const void* bias, int mode, int out_dtype, void* out, int T, int N, int K) {
  if (a_dtype == kF32 && w_dtype == kF32)
    return launch_generic_bias<float, float>(s, a, w, bias_dtype, bias, mode, out_dtype, out, T, N, K);
  if (a_dtype == kF32 && w_dtype == kBF16)
    return launch_generic_bias<float, bf16_t>(s, a, w, bias_dtype, bias, mode, out_dtype, out, T, N, K);
  if (a_dtype == kBF16 && w_dtype == kF32)
    return launch_generic_bias<bf16_t, float>(s, a, w, bias_dtype, bias, mode, out_dtype, out, T, N, K);
  return launch_generic_bias<bf16_t, bf16_t>(s, a, w, bias_dtype, bias, mode, out_dtype, out, T, N, K);
}

}  // namespace sprout
