// What a block of the tiled products does with its sums.  Waves in a (waves / WAVES_N) x WAVES_N arrangement
// (2 x 2 unless said otherwise), each holding WM x WN tiles of 32 x 32 from 32x32x16 MFMA with the weights as the A operand: lane (li = lane % 32,
// lk = lane / 32) holds out[t = tile row li][n = tile column 8 * (r / 4) + 4 * lk + r % 4] in element r.
#pragma once
#include "mfma.h"

namespace sprout {

enum { kStore = 0, kAccumulate = 1, kStoreF32 = 2, kSilu = 3 };   // kSilu: gate rows and up rows, see below

// Orders a wave's LDS writes before its own later reads of what other lanes wrote (and the reverse).
__device__ __forceinline__ void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// `turn` is LDS that no wave of the block reads or fills any more, at least waves * 32 * (32 WN + 4) floats;
// it is used only when K is split over blocks (gridDim.z > 1).
template <int WM, int WN, int MODE, typename TB, int WAVES_N = 2>
__device__ __forceinline__ void tile_epilogue(floatx16 (&acc)[WM][WN], float* turn_all, const TB* __restrict__ bias,
                                              void* __restrict__ out, int T, int N, int t0, int n0) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int li = lane & 31, lk = lane >> 5;
  if (MODE == kSilu) {
    // tile columns 2 m of a wave hold gate rows, columns 2 m + 1 the matching up rows:
    // out[t, n] = silu(gate) * up, both rounded to bfloat16 first, as where they are stored before the gated product
    static_assert(MODE != kSilu || WN % 2 == 0, "the gated epilogue pairs tile columns");
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      const int t = t0 + (wm * WM + i) * 32 + li;
      if (t >= T) continue;
#pragma unroll
      for (int m = 0; m < WN / 2; ++m) {
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const int n = n0 / 2 + (wn * (WN / 2) + m) * 32 + 8 * rg + 4 * lk;
          if (n >= N) continue;
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float g = to_float(bf16_t{f32_to_bf16_bits(acc[i][2 * m][4 * rg + r])});
            const float u = to_float(bf16_t{f32_to_bf16_bits(acc[i][(2 * m + 1) % WN][4 * rg + r])});
            v[r] = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u;
          }
          uint16_t* dst = reinterpret_cast<uint16_t*>(out) + size_t(t) * N + n;
          if (n + 4 <= N && (N & 3) == 0) *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
          else for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = f32_to_bf16_bits(v[r]);
        }
      }
    }
    return;
  }

  if (MODE == kAccumulate && gridDim.z > 1) {
    // K is split over blocks: the partial sums are added with float atomics.  A lane holds four n of one
    // token, so 64 lanes would touch 32 rows of the output at once; each wave turns its tiles round in
    // its own quarter of the LDS first, and then adds whole rows (64 consecutive floats per instruction).
    constexpr int PITCH = WN * 32 + 4;
    float* turn = turn_all + wave * 32 * PITCH;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg)
          *reinterpret_cast<float4*>(turn + li * PITCH + j * 32 + 8 * rg + 4 * lk) =
              make_float4(acc[i][j][4 * rg], acc[i][j][4 * rg + 1], acc[i][j][4 * rg + 2], acc[i][j][4 * rg + 3]);
      wave_lds_fence();
      const int tbase = t0 + (wm * WM + i) * 32, nbase = n0 + wn * WN * 32;
      for (int tr = 0; tr < 32 && tbase + tr < T; ++tr)
#pragma unroll
        for (int c = 0; c < WN * 32; c += 64) {
          const int col = c + lane;
          if (col < WN * 32 && nbase + col < N) {
            float v = turn[tr * PITCH + col];
            if (bias && blockIdx.z == 0) v += to_float(bias[nbase + col]);
            unsafeAtomicAdd(reinterpret_cast<float*>(out) + size_t(tbase + tr) * N + nbase + col, v);
          }
        }
      wave_lds_fence();
    }
    return;
  }

  // lane holds out[t = tile row li][n = tile column 8 * (r / 4) + 4 * lk + r % 4]: four consecutive n per group
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int t = t0 + (wm * WM + i) * 32 + li;
    if (t >= T) continue;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int n = n0 + (wn * WN + j) * 32 + 8 * rg + 4 * lk;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
          v[r] = acc[i][j][4 * rg + r] + ((bias && blockIdx.z == 0 && n + r < N) ? to_float(bias[n + r]) : 0.f);
        const size_t o = size_t(t) * N + n;
        const bool whole = n + 4 <= N && (N & 3) == 0;
        if (MODE == kStore) {
          uint16_t* dst = reinterpret_cast<uint16_t*>(out) + o;
          if (whole) *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
          else for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = f32_to_bf16_bits(v[r]);
        } else if (MODE == kStoreF32) {
          float* dst = reinterpret_cast<float*>(out) + o;
          if (whole) *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
          else for (int r = 0; r < 4 && n + r < N; ++r) dst[r] = v[r];
        } else {
          float* dst = reinterpret_cast<float*>(out) + o;
          if (whole) {
            const float4 old = *reinterpret_cast<float4*>(dst);
            *reinterpret_cast<float4*>(dst) = make_float4(old.x + v[0], old.y + v[1], old.z + v[2], old.w + v[3]);
          } else {
            for (int r = 0; r < 4 && n + r < N; ++r) dst[r] += v[r];
          }
        }
      }
    }
  }
}

}  // namespace sprout
