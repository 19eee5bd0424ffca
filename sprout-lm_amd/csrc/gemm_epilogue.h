// What a block of the tiled products does with its sums.  Waves in a (waves / WAVES_N) x WAVES_N arrangement
// (2 x 2 unless said otherwise), each holding WM x WN tiles of 32 x 32 from 32x32x16 MFMA with the weights as the A operand: lane (li = lane % 32,
// lk = lane / 32) holds out[t = tile row li][n = tile column 8 * (r / 4) + 4 * lk + r % 4] in element r.
#pragma once
#include "mfma.h"

namespace sprout {

enum { kStore = 0, kAccumulate = 1, kStoreF32 = 2, kSilu = 3, kRope = 4 };   // kSilu, kRope: see below

// What the rotating epilogue (kRope) needs beside the product: the rows of w are q, k and v heads of size hd.
struct RopeArgs {
  const int32_t* positions;      // [T]
  const float* inv_freq;         // [hd / 2]
  const int32_t* slot_mapping;   // [T]: page * page_size + slot of the token's key and value, or -1
  uint16_t* k_pool;              // [page][kv head][slot][dim]
  uint16_t* v_pool;              // [page][kv head][dim][slot]
  int nq, nkv, hd, page_size;
  const float2* table;           // [T][hd / 2] (cosine, sine) of positions[t] * inv_freq[d], or null: computed here
};

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
                                              void* __restrict__ out, int T, int N, int t0, int n0,
                                              const RopeArgs& rope = RopeArgs{}) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int li = lane & 31, lk = lane >> 5;
  if (MODE == kRope) {
    // Tile columns come in groups of 64: 32 dimensions of a head's first half (tile column 2 m of a wave) and
    // their rotation partners, half a head further on (tile column 2 m + 1), so that a lane holds both of a pair.
    // Bias, rounding to bfloat16 (as where the projections pass through memory), rotation of q and k heads;
    // q goes to out [T, nq * hd], k and v into the paged pools.
    static_assert(MODE != kRope || WN % 2 == 0, "the rotating epilogue pairs tile columns");
    const int hd = rope.hd, half = hd / 2, groups_per_head = half / 32, heads = rope.nq + 2 * rope.nkv;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      const int t = t0 + (wm * WM + i) * 32 + li;
      if (t >= T) continue;
      const float pos = float(rope.positions[t]);
      const int slot = rope.slot_mapping[t];
      const int page = slot >= 0 ? slot / rope.page_size : 0, off = slot >= 0 ? slot % rope.page_size : 0;
#pragma unroll
      for (int m = 0; m < WN / 2; ++m) {
        const int group = n0 / 64 + wn * (WN / 2) + m, head = group / groups_per_head, u = group % groups_per_head;
        if (head >= heads) continue;
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const int d0 = 32 * u + 8 * rg + 4 * lk;          // four consecutive dimensions of the first half
          float lo[4], hi[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int n = head * hd + d0 + r;
            float a = acc[i][2 * m][4 * rg + r], b = acc[i][(2 * m + 1) % WN][4 * rg + r];
            if (bias) { a += to_float(bias[n]); b += to_float(bias[n + half]); }
            a = to_float(bf16_t{f32_to_bf16_bits(a)});
            b = to_float(bf16_t{f32_to_bf16_bits(b)});
            if (head < rope.nq + rope.nkv) {
              float sn, cs;
              if (rope.table) {
                const float2 e = rope.table[size_t(t) * half + d0 + r];
                cs = e.x;
                sn = e.y;
              } else {
                sincosf(pos * rope.inv_freq[d0 + r], &sn, &cs);
              }
              lo[r] = a * cs - b * sn;
              hi[r] = b * cs + a * sn;
            } else {
              lo[r] = a;
              hi[r] = b;
            }
          }
          const uint2 blo = make_uint2(pack_bf16x2(lo[0], lo[1]), pack_bf16x2(lo[2], lo[3]));
          const uint2 bhi = make_uint2(pack_bf16x2(hi[0], hi[1]), pack_bf16x2(hi[2], hi[3]));
          if (head < rope.nq) {
            uint16_t* q = reinterpret_cast<uint16_t*>(out) + size_t(t) * (size_t(rope.nq) * hd) + head * hd + d0;
            *reinterpret_cast<uint2*>(q) = blo;
            *reinterpret_cast<uint2*>(q + half) = bhi;
          } else if (slot >= 0) {
            if (head < rope.nq + rope.nkv) {
              uint16_t* k = rope.k_pool + ((size_t(page) * rope.nkv + (head - rope.nq)) * rope.page_size + off) * hd + d0;
              *reinterpret_cast<uint2*>(k) = blo;
              *reinterpret_cast<uint2*>(k + half) = bhi;
            } else {
              uint16_t* v = rope.v_pool + (size_t(page) * rope.nkv + (head - rope.nq - rope.nkv)) * hd * rope.page_size + off;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                v[size_t(d0 + r) * rope.page_size] = f32_to_bf16_bits(lo[r]);
                v[size_t(d0 + half + r) * rope.page_size] = f32_to_bf16_bits(hi[r]);
              }
            }
          }
        }
      }
    }
    return;
  }
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
