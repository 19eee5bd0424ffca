// Skinny bfloat16 products for decoding (T <= 64) with the work of the neighbouring small kernels
// folded in.  One block of four waves owns NT tiles of 16 weight rows; the waves split K between
// them (64 elements at a time, interleaved), so that even a matrix with few rows keeps many loads in
// flight, and their partial sums meet in LDS.  What can be folded in:
//   prologue  NORM   the activations are RMSNorm(residual) * weight, computed by the block itself from the
//                    float32 residual, 16 tokens a block (further tokens are further blocks along the grid's
//                    z).  A lane asks for its token's values of the wave's steps before the weights; the
//                    squares of the four waves meet in LDS while the weights are on their way, and the lanes
//                    then turn (x * scale) * weight into matrix-core operands in registers: the numbers that
//                    the norm kernel would have stored, so a token's activations do not depend on which of
//                    the two ways a step takes.
//   epilogue  kEpiStore / kEpiAccumulate / kEpiStoreF32   as the plain product (+ bias)
//             kEpiRope   the block's rows are `rows_per_block` rotation pairs (dims d and d + head/2 of a head,
//                        counted through all heads): their first rows in one tile and their partners in the other
//                        (up to 16 pairs), or both in one gathered tile (NT = 1, up to 8 pairs: rows 0-7 and
//                        8-15); the pairs a block takes are chosen so that the blocks are a whole number per CU
//                        where they can be (a CU pulls its rows no faster for having them in fewer blocks); adds
//                        the bias, rotates q and k heads, writes q and scatters k, v into the paged cache
//             kEpiSilu   the block owns `rows_per_block` inner columns: their gate rows and the matching up rows
//                        fill its tiles one after the other (two tiles hold 16 of each; three hold up to 24, which
//                        lets a matrix be cut into a whole number of blocks per CU); writes silu(gate) * up
// Accumulating products may also be split along K over several blocks (hardware float atomics).
//
// A step of decoded tokens spends a few microseconds in each of these kernels, and a wave's every vector
// instruction is four cycles of them: with K in whole steps of 64 (K64) the loads carry no bounds of their
// own, whole steps are switched by scalar branches, and addresses are one base per pass plus constants.
#include "mfma.h"
#include "sprout_hip.h"

namespace sprout {

enum { kEpiStore = 0, kEpiAccumulate = 1, kEpiStoreF32 = 2, kEpiRope = 3, kEpiSilu = 4 };

struct FusedArgs {
  const uint16_t* x;         // activations [T, K] bfloat16 (without NORM)
  const float* residual;     // float32 [T, K] (with NORM)
  const void* norm_w;        // [K]
  int norm_w_bf16;
  float eps;
  const uint16_t* w;         // [N, K]
  const void* bias;          // [N] or null
  int bias_bf16;
  void* out;                 // [T, N] (store / accumulate); [T, N / 2] for kEpiSilu; q rows [T, nq * hd] for kEpiRope
  int T, N, K, k_per_split;
  int partner;               // rows between a row and its partner (kEpiRope: hd / 2, kEpiSilu: N / 2)
  int rows_per_block;        // kEpiSilu: inner columns a block owns (at most 8 * NT); kEpiRope: rotation pairs a block owns
  // kEpiRope
  const int32_t* positions;
  const float* inv_freq;
  const int32_t* slot_mapping;
  uint16_t* k_pool;
  uint16_t* v_pool;
  int nq, nkv, hd, page_size, rotary_dim;
  int page_shift;            // page_size == 1 << page_shift, or -1 where it is no power of two
};

// A bias value as it lies in memory (bfloat16 bits or float32 bits), and its value.  The two are kept apart
// because turning the bits into a number waits for the load, and loads return in the order of their requests:
// done where the bias is asked for, it would wait for the weights asked for before it.
__device__ __forceinline__ uint32_t load_param_bits(const void* p, int is_bf16, int i) {
  return is_bf16 ? uint32_t(reinterpret_cast<const uint16_t*>(p)[i]) : reinterpret_cast<const uint32_t*>(p)[i];
}
__device__ __forceinline__ float param_value(uint32_t bits, int is_bf16) {
  return __uint_as_float(is_bf16 ? bits << 16 : bits);
}

__device__ __forceinline__ float4 ldg_f4(const float* __restrict__ p) { return *reinterpret_cast<const float4*>(p); }

// The norm prologue's inputs of one pass as they come from memory: for each of the wave's UN steps the lane's 16
// values of its token (two groups of 8 along K) and the norm's weights for them.  `request` asks for all of
// them; `squares` sums the squares of x; `operands` turns them into (x * scale) * norm weight in bfloat16, the
// very numbers that the norm kernel stores.
// `row` and `norm_w` point at the lane's first value of the pass (step s0); step s0 + 4 u lies 256 u values on.
// K64: K is whole steps, a step is there or not for the whole wave (`steps_left` of them from s0 on, every
// fourth).  Otherwise groups past the end of K are read from `safe_row` / `safe_w` instead (valid addresses:
// the starts of the row and of the norm's weights) and count for nothing.
template <int UN, bool K64>
struct NormInputs {
  float4 xf[UN][2][2];
  uint4 nw[UN][2][2];   // the norm's weights as stored: 8 bfloat16 in [0], or 8 float32 in [0] and [1]

  __device__ __forceinline__ void request(const float* __restrict__ row, const void* __restrict__ norm_w, bool BF,
                                          int steps_left, int k_left, const float* __restrict__ safe_row,
                                          const void* __restrict__ safe_w) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (K64 && 4 * u >= steps_left) {   // the same for every lane of the wave: a scalar branch
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          xf[u][h][0] = xf[u][h][1] = make_float4(0.f, 0.f, 0.f, 0.f);
          nw[u][h][0] = nw[u][h][1] = make_uint4(0, 0, 0, 0);
        }
        continue;
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int at = 256 * u + 8 * h;
        const bool there = K64 || (4 * u < steps_left && at < k_left);
        const float* xp = there ? row + at : safe_row;
        xf[u][h][0] = ldg_f4(xp);
        xf[u][h][1] = ldg_f4(xp + 4);
        nw[u][h][1] = make_uint4(0, 0, 0, 0);
        if (BF) {
          nw[u][h][0] = ldg128(there ? reinterpret_cast<const uint16_t*>(norm_w) + at : reinterpret_cast<const uint16_t*>(safe_w));
        } else {
          const float* wp = there ? reinterpret_cast<const float*>(norm_w) + at : reinterpret_cast<const float*>(safe_w);
          nw[u][h][0] = ldg128(wp);
          nw[u][h][1] = ldg128(wp + 4);
        }
      }
    }
  }

  // This lane's share of the sum of squares of its token over the pass.
  __device__ __forceinline__ float squares(int steps_left, int k_left) const {
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float4 x0 = xf[u][h][0], x1 = xf[u][h][1];
        float sq = fmaf(x0.x, x0.x, fmaf(x0.y, x0.y, fmaf(x0.z, x0.z, x0.w * x0.w)));
        sq = fmaf(x1.x, x1.x, fmaf(x1.y, x1.y, fmaf(x1.z, x1.z, fmaf(x1.w, x1.w, sq))));
        if (K64) sum += sq;                     // a step that is not there holds zeros
        else sum = fmaf((4 * u < steps_left && 256 * u + 8 * h < k_left) ? 1.f : 0.f, sq, sum);
      }
    return sum;
  }

  // (a group past the end of K meets weights of the product that are zeros: what stands here for it does not count)
  __device__ __forceinline__ void operands(bool BF, float scale, uint4 (&xb)[UN][1][2]) const {
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float4 x0 = xf[u][h][0], x1 = xf[u][h][1];
        float4 w0, w1;
        const uint4 b = nw[u][h][0], c = nw[u][h][1];
        if (BF) {
          w0 = make_float4(__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u),
                           __uint_as_float(b.y << 16), __uint_as_float(b.y & 0xffff0000u));
          w1 = make_float4(__uint_as_float(b.z << 16), __uint_as_float(b.z & 0xffff0000u),
                           __uint_as_float(b.w << 16), __uint_as_float(b.w & 0xffff0000u));
        } else {
          w0 = make_float4(__uint_as_float(b.x), __uint_as_float(b.y), __uint_as_float(b.z), __uint_as_float(b.w));
          w1 = make_float4(__uint_as_float(c.x), __uint_as_float(c.y), __uint_as_float(c.z), __uint_as_float(c.w));
        }
        xb[u][0][h] = make_uint4(pack_bf16x2((x0.x * scale) * w0.x, (x0.y * scale) * w0.y),
                                 pack_bf16x2((x0.z * scale) * w0.z, (x0.w * scale) * w0.w),
                                 pack_bf16x2((x1.x * scale) * w1.x, (x1.y * scale) * w1.y),
                                 pack_bf16x2((x1.z * scale) * w1.z, (x1.w * scale) * w1.w));
      }
  }
};

// The weight row that lane-row `lr` of tile `i` of block `b` multiplies (an existing row also where the tile
// has no row for the lane: what it computes there is not used, and in the gated product's last tile, which the
// block's rows fill only in part, such a lane asks for nothing).
template <int EPI, int NT>
__device__ __forceinline__ int weight_row(const FusedArgs& a, int b, int i, int lr) {
  int row;
  if (EPI == kEpiRope) {
    // pair p of all heads' pairs is dimension p % (hd / 2) of head p / (hd / 2) and its partner half a head on;
    // one gathered tile: rows 0..7 are the block's pairs' first rows, rows 8..15 their partners
    const int slot = NT == 1 ? (lr & 7) : lr, second = NT == 1 ? lr >> 3 : i;
    const int pair = b * a.rows_per_block + slot;
    row = (pair / a.partner) * a.hd + pair % a.partner + second * a.partner;
  } else if (EPI == kEpiSilu) {
    // the block's gate rows, then its up rows, fill the tiles one after the other
    const int slot = 16 * i + lr, r = a.rows_per_block;
    row = slot < r ? b * r + slot : a.partner + b * r + slot - r;
  } else {
    row = 16 * (NT * b + i) + lr;
  }
  return min(a.N - 1, row);
}

template <int TN, int EPI, bool NORM, int NT, bool K64, int UN>
__global__ __launch_bounds__(256) void gemm_fused_kernel(FusedArgs a) {
  static_assert(NT == 2 || EPI == kEpiRope || EPI == kEpiSilu, "one or three tiles a block only where rows are paired");
  static_assert(!NORM || TN == 1, "the norm prologue takes one tile of 16 tokens");
  extern __shared__ uint4 lds[];
  // reduction buffer [4 waves][NT tiles][TN][64 lanes] float4, then (NORM) sums of squares [4 waves][16 tokens]
  float4* red = reinterpret_cast<float4*>(lds);
  float* squares = reinterpret_cast<float*>(lds + 4 * NT * TN * 64);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same for the whole wave: a scalar
  const int lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  const int t0 = blockIdx.z * (16 * TN);   // the block's first token: tiles of tokens lie along z
  const int k_begin = blockIdx.y * a.k_per_split;
  const int k_end = min(a.K, k_begin + a.k_per_split);
  const int steps = (k_end - k_begin + 63) / 64;

  // the lane's first weight of each tile, and of the activations, at step 0
  const uint16_t* wrow[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) wrow[i] = a.w + size_t(weight_row<EPI, NT>(a, blockIdx.x, i, lr)) * a.K + k_begin + 16 * lj;
  const float* norm_row = NORM ? a.residual + size_t(min(t0 + lr, a.T - 1)) * a.K + k_begin + 16 * lj : nullptr;
  const char* norm_w0 = NORM ? reinterpret_cast<const char*>(a.norm_w) + size_t(k_begin + 16 * lj) * (a.norm_w_bf16 ? 2 : 4) : nullptr;
  const uint16_t* xrow[TN];
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)   // rows past T repeat the last one: their sums are not used
    xrow[tn] = NORM ? nullptr : a.x + size_t(min(t0 + tn * 16 + lr, a.T - 1)) * a.K + k_begin + 16 * lj;

  // The weights' way from memory is the longest wait of the kernel: they are requested at once, UN steps
  // of this wave together (steps s0, s0 + 4, ...).
  // UN: steps of 64 requested together (a pass of the four waves is 4 UN steps): 4, 2 with four token tiles
  // (registers), 8 where a block has a CU to itself and a long K, so that fewer trips to memory follow each other
  // Whether this lane's row of tile i is one of the block's rows: the gated product's last tile and the rotating
  // product's tiles may be filled in part, and a lane without a row asks for nothing.
  bool row_there[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    if (EPI == kEpiSilu) {
      row_there[i] = 16 * i + lr < 2 * a.rows_per_block;
    } else if (EPI == kEpiRope) {
      const int slot = NT == 1 ? (lr & 7) : lr;
      row_there[i] = slot < a.rows_per_block && int(blockIdx.x) * a.rows_per_block + slot < a.N / a.hd * a.partner;
    } else {
      row_there[i] = true;
    }
  }
  uint4 wa[UN][NT][2];
  auto load_weights = [&](int s0) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const bool step_there = s0 + 4 * u < steps;
      if (K64) {
        if (step_there) {   // a scalar branch
#pragma unroll
          for (int i = 0; i < NT; ++i) {
            if (((EPI == kEpiSilu && NT == 3 && i == 2) || EPI == kEpiRope) && !row_there[i]) {
              wa[u][i][0] = wa[u][i][1] = make_uint4(0, 0, 0, 0);
              continue;
            }
            wa[u][i][0] = ldg128(wrow[i] + 64 * s0 + 256 * u);
            wa[u][i][1] = ldg128(wrow[i] + 64 * s0 + 256 * u + 8);
          }
        } else {
#pragma unroll
          for (int i = 0; i < NT; ++i) wa[u][i][0] = wa[u][i][1] = make_uint4(0, 0, 0, 0);
        }
      } else {
        const int k = k_begin + 64 * (s0 + 4 * u) + 16 * lj;
        const bool in0 = step_there && k < k_end, in1 = step_there && k + 8 < k_end;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          wa[u][i][0] = in0 && row_there[i] ? ldg128(wrow[i] + 64 * s0 + 256 * u) : make_uint4(0, 0, 0, 0);
          wa[u][i][1] = in1 && row_there[i] ? ldg128(wrow[i] + 64 * s0 + 256 * u + 8) : make_uint4(0, 0, 0, 0);
        }
      }
    }
  };
  // The norm prologue's rows are requested right after the weights; both are then on their way together.
  NormInputs<NORM ? UN : 1, K64> normed;
  auto request_rows = [&](int s0) {
    normed.request(norm_row + 64 * s0, norm_w0 + size_t(64 * s0) * (a.norm_w_bf16 ? 2 : 4), a.norm_w_bf16, steps - s0,
                   k_end - (k_begin + 16 * lj + 64 * s0), a.residual, a.norm_w);
  };
  // NORM: the rows first (they come from the caches and are needed first: their sum of squares is exchanged
  // between the waves while the weights, which take longest, are on their way)
  if constexpr (NORM) request_rows(wave);
  load_weights(wave);
  __builtin_amdgcn_sched_barrier(0);   // keep these requests ahead of everything below
  // What the epilogue reads per output (bias, position, rotation frequency, cache slot) is requested now
  // as well: asked for after the sums are done, it would be one more trip to memory at the end of the kernel.
  // thread -> (token et of a tile, row ei of a tile), as in the epilogue below
  const int et = threadIdx.x >> 4, ei = threadIdx.x & 15;
  const int er = (EPI == kEpiRope && NT == 1) ? (ei & 7) : ei;   // one gathered tile: threads ei < 8 own a dimension and its partner
  // the output rows this thread finishes: kEpiRope dimension er of the block and its partner; kEpiSilu the
  // block's inner columns ei and 16 + ei; otherwise row ei of either tile
  constexpr int OUTS = EPI == kEpiSilu ? (NT + 1) / 2 : 2;
  // the plain epilogues: thread -> (row pr of the block's 32, tokens pt and pt + 8 of a tile of 16), so that a
  // wave stores or adds runs of 32 neighbouring numbers of a token's row
  constexpr bool PLAIN = EPI == kEpiStore || EPI == kEpiAccumulate || EPI == kEpiStoreF32;
  const int pr = threadIdx.x & 31, pt = threadIdx.x >> 5;
  uint32_t bias_bits[2] = {0u, 0u};   // zero bits are zero in either dtype
  if (PLAIN) {
    if (a.bias && blockIdx.y == 0 && 32 * int(blockIdx.x) + pr < a.N)
      bias_bits[0] = load_param_bits(a.bias, a.bias_bf16, 32 * blockIdx.x + pr);
  }
  int position_of[TN], slot_of[TN];
  float frequency = 0.f;
  int rope_head = 0, rope_dim = 0;
  bool rope_pair = false;          // this thread finishes a pair of the block
  if (EPI == kEpiRope) {
    const int pair = blockIdx.x * a.rows_per_block + er;
    rope_pair = (NT == 2 || ei < 8) && er < a.rows_per_block && pair < a.N / a.hd * a.partner;
    rope_head = rope_pair ? pair / a.partner : 0;
    rope_dim = rope_pair ? pair - rope_head * a.partner : 0;   // < hd / 2; the partner is hd / 2 further
    if (rope_pair && a.bias) {
      bias_bits[0] = load_param_bits(a.bias, a.bias_bf16, rope_head * a.hd + rope_dim);
      bias_bits[1] = load_param_bits(a.bias, a.bias_bf16, rope_head * a.hd + rope_dim + a.partner);
    }
    if (rope_dim < a.rotary_dim / 2) frequency = a.inv_freq[rope_dim];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int t = min(t0 + tn * 16 + et, a.T - 1);
      position_of[tn] = a.positions[t];
      slot_of[tn] = a.slot_mapping[t];
    }
  }

  floatx4 acc[NT][TN];
#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) acc[i][tn] = floatx4{0.f, 0.f, 0.f, 0.f};

  // NORM: 1 / sqrt(mean(x^2) + eps) of token lr, before anything is rounded: the activations are then the numbers
  // that the norm kernel stores, whichever way a step is computed.  The four waves hold a quarter of the row's
  // steps each; rows longer than one pass (4 UN steps) are read once more for their squares.  The weights asked
  // for above are on their way meanwhile.
  float row_scale = 1.f;
  if constexpr (NORM) {
    float square_sum = normed.squares(steps - wave, k_end - (k_begin + 16 * lj + 64 * wave));
    for (int s0 = wave + 4 * UN; s0 < steps; s0 += 4 * UN) {
      NormInputs<UN, K64> further;
      further.request(norm_row + 64 * s0, norm_w0 + size_t(64 * s0) * (a.norm_w_bf16 ? 2 : 4), a.norm_w_bf16, steps - s0,
                      k_end - (k_begin + 16 * lj + 64 * s0), a.residual, a.norm_w);
      square_sum += further.squares(steps - s0, k_end - (k_begin + 16 * lj + 64 * s0));
    }
    square_sum += __shfl_xor(square_sum, 16, 64);   // the four lanes of a token hold a quarter of the wave's steps each
    square_sum += __shfl_xor(square_sum, 32, 64);
    if (lj == 0) squares[wave * 16 + lr] = square_sum;
    __syncthreads();
    row_scale = 1.0f / sqrtf((squares[lr] + squares[16 + lr] + squares[32 + lr] + squares[48 + lr]) / float(a.K) + a.eps);
  }

  // this wave's steps of 64 along K: wave, wave + 4, ...; UN steps are loaded before they are multiplied
  for (int s0 = wave; s0 < steps; s0 += 4 * UN) {
    if (s0 != wave) {
      load_weights(s0);
      if constexpr (NORM) request_rows(s0);
    }
    uint4 xb[UN][TN][2];
    if constexpr (NORM) {
      // Lane (lr, lj) needs 16 values of token lr per step, as the matrix cores take them.  They come straight
      // from the float32 residual, times the token's scale, times the norm's weights, rounded to bfloat16.
      normed.operands(a.norm_w_bf16, row_scale, xb);
    } else {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const bool step_there = s0 + 4 * u < steps;
        const int k = k_begin + 64 * (s0 + 4 * u) + 16 * lj;
        const bool in0 = step_there && (K64 || k < k_end), in1 = step_there && (K64 || k + 8 < k_end);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
          if (K64) {
            if (step_there) {
              xb[u][tn][0] = ldg128(xrow[tn] + 64 * s0 + 256 * u);
              xb[u][tn][1] = ldg128(xrow[tn] + 64 * s0 + 256 * u + 8);
            } else {
              xb[u][tn][0] = xb[u][tn][1] = make_uint4(0, 0, 0, 0);
            }
          } else {
            xb[u][tn][0] = in0 ? ldg128(xrow[tn] + 64 * s0 + 256 * u) : make_uint4(0, 0, 0, 0);
            xb[u][tn][1] = in1 ? ldg128(xrow[tn] + 64 * s0 + 256 * u + 8) : make_uint4(0, 0, 0, 0);
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UN; ++u)
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          acc[i][tn] = mfma16(as_bf16x8(wa[u][i][0]), as_bf16x8(xb[u][tn][0]), acc[i][tn]);
          acc[i][tn] = mfma16(as_bf16x8(wa[u][i][1]), as_bf16x8(xb[u][tn][1]), acc[i][tn]);
        }
  }

#pragma unroll
  for (int i = 0; i < NT; ++i)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
      red[((wave * NT + i) * TN + tn) * 64 + lane] = make_float4(acc[i][tn][0], acc[i][tn][1], acc[i][tn][2], acc[i][tn][3]);
  __syncthreads();

  // The sum of the four waves for (tile, row of the tile, token tile tn, token et): row r of a tile lies in
  // MFMA lane (r / 4) * 16 + token, element r % 4.
  auto summed_at = [&](int tile, int row, int tn, int token) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w)
      sum += reinterpret_cast<const float*>(&red[((w * NT + tile) * TN + tn) * 64 + (row >> 2) * 16 + token])[row & 3];
    return sum;
  };
  auto summed = [&](int tile, int row, int tn) { return summed_at(tile, row, tn, et); };
#pragma unroll
  for (int tn = 0; tn < TN; ++tn) {
    const int t = t0 + tn * 16 + et;
    if (EPI == kEpiSilu) {
      const int r = a.rows_per_block;
#pragma unroll
      for (int o = 0; o < OUTS; ++o) {
        const int p = 16 * o + ei, n = blockIdx.x * r + p;     // inner column p of the block
        if (p >= r || n >= a.partner || t >= a.T) continue;
        const int gate = p, up = p + r;                         // their places among the block's rows
        const float gv = summed(gate >> 4, gate & 15, tn), uv = summed(up >> 4, up & 15, tn);
        // the engine keeps gate and up as bfloat16 before the gated product; keep the same roundings
        const float g = to_float(bf16_t{f32_to_bf16_bits(gv)}), u = to_float(bf16_t{f32_to_bf16_bits(uv)});
        reinterpret_cast<uint16_t*>(a.out)[size_t(t) * a.partner + n] = f32_to_bf16_bits(g / (1.0f + expf(-g)) * u);
      }
      continue;
    }
    if (PLAIN) {
      static_assert(!PLAIN || NT == 2, "the plain epilogues take blocks of two tiles");
      const int n = 32 * blockIdx.x + pr;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int token = pt + 8 * j, tp = t0 + tn * 16 + token;
        if (tp >= a.T || n >= a.N) continue;
        const float v = summed_at(pr >> 4, pr & 15, tn, token) + param_value(bias_bits[0], a.bias_bf16);
        const size_t o = size_t(tp) * a.N + n;
        if (EPI == kEpiStore) reinterpret_cast<uint16_t*>(a.out)[o] = f32_to_bf16_bits(v);
        else if (EPI == kEpiStoreF32) reinterpret_cast<float*>(a.out)[o] = v;
        else if (gridDim.y == 1) reinterpret_cast<float*>(a.out)[o] += v;
        else unsafeAtomicAdd(reinterpret_cast<float*>(a.out) + o, v);
      }
      continue;
    }
    float v[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const float sum = (EPI == kEpiRope && NT == 1) ? summed(0, er + 8 * i, tn) : summed(i, ei, tn);
      v[i] = sum + param_value(bias_bits[i], a.bias_bf16);
    }
    if (t >= a.T || (EPI == kEpiRope && !rope_pair)) continue;
    {  // kEpiRope
      const int head = rope_head, d = rope_dim;      // d < hd / 2; partner dim d + hd / 2
      // projections are kept as bfloat16 before the rotation, as in the unfused path
      float lo = to_float(bf16_t{f32_to_bf16_bits(v[0])}), hi = to_float(bf16_t{f32_to_bf16_bits(v[1])});
      const int half = a.hd / 2;
      if (head < a.nq + a.nkv && d < a.rotary_dim / 2 && half == a.rotary_dim / 2) {
        float sn, cs;
        sincosf(float(position_of[tn]) * frequency, &sn, &cs);
        const float rl = lo * cs - hi * sn, rh = hi * cs + lo * sn;
        lo = rl;
        hi = rh;
      }
      const uint16_t blo = f32_to_bf16_bits(lo), bhi = f32_to_bf16_bits(hi);
      if (head < a.nq) {
        uint16_t* q = reinterpret_cast<uint16_t*>(a.out) + size_t(t) * (size_t(a.nq) * a.hd) + head * a.hd;
        q[d] = blo;
        q[d + half] = bhi;
      } else {
        const int slot = slot_of[tn];
        if (slot >= 0) {
          int page, off;
          if (a.page_shift >= 0) {      // the same for every thread: a scalar branch, and no division
            page = slot >> a.page_shift;
            off = slot & (a.page_size - 1);
          } else {
            page = slot / a.page_size;
            off = slot % a.page_size;
          }
          if (head < a.nq + a.nkv) {
            uint16_t* k = a.k_pool + ((size_t(page) * a.nkv + (head - a.nq)) * a.page_size + off) * a.hd;
            k[d] = blo;
            k[d + half] = bhi;
          } else {
            uint16_t* vp = a.v_pool + (size_t(page) * a.nkv + (head - a.nq - a.nkv)) * a.hd * a.page_size + off;
            vp[size_t(d) * a.page_size] = blo;
            vp[size_t(d + half) * a.page_size] = bhi;
          }
        }
      }
    }
  }
}

static size_t fused_lds_bytes(int TN, bool norm, int NT = 2) {
  return sizeof(float4) * 4 * NT * TN * 64 + (norm ? sizeof(float) * 4 * 16 : 0);
}

template <int TN, int EPI, bool NORM, int NT, int UN>
static int launch_fused_un(hipStream_t s, const FusedArgs& a, int blocks, int splits) {
  const size_t lds = fused_lds_bytes(TN, NORM, NT);     // at most 48 KB (four token tiles of three tiles)
  const dim3 grid(blocks, splits, (a.T + 16 * TN - 1) / (16 * TN));   // z: the tokens in tiles of 16 TN
  if (a.K % 64 == 0 && a.k_per_split % 64 == 0)
    gemm_fused_kernel<TN, EPI, NORM, NT, true, UN><<<grid, 256, lds, s>>>(a);
  else
    gemm_fused_kernel<TN, EPI, NORM, NT, false, UN><<<grid, 256, lds, s>>>(a);
  return check_launch("sp_gemm_fused");
}

template <int TN, int EPI, bool NORM, int NT = 2>
static int launch_fused(hipStream_t s, const FusedArgs& a, int blocks, int splits) {
  if constexpr (TN == 1 && !NORM && NT <= 2) {
    // Few blocks with a long K each: a block alone on its CU hides no trip to memory behind another block's, so
    // its waves ask for twice the steps at once and make half the trips (registers allow it without the norm's
    // inputs; 28 heads of 128 at a width of 3,584: four passes become two).
    const int steps_a_wave = (min(a.K, a.k_per_split) + 255) / 256;
    if (blocks * splits * ((a.T + 15) / 16) <= 256 && steps_a_wave > 4)
      return launch_fused_un<TN, EPI, NORM, NT, 8>(s, a, blocks, splits);
  }
  return launch_fused_un<TN, EPI, NORM, NT, TN >= 4 ? 2 : 4>(s, a, blocks, splits);
}

// Rotation pairs a block of the q/k/v product owns (all heads' pairs are counted through: a block may end in one
// head and go on in the next).  A CU pulls its rows at about the same rate however many blocks it holds, and no
// faster for having more of them in flight, so the rows are cut for the CU that gets the most: bytes a block asks
// for (two rows a pair, and the activations, which every block reads whole) times blocks per CU, rounded up.  Up
// to 8 pairs lie in one gathered tile, up to 16 in two.  (Blocks of 8 or 16 pairs whatever the sizes: 18 heads of
// 64 at a width of 896, 8 tokens: 72 blocks; 36 heads of 128 at 3,584: 144 blocks on 256 CUs.)
static int rope_pairs_per_block(int T, int N, int K, bool norm) {
  const int pairs = N / 2, token_tiles = norm ? (T + 15) / 16 : 1;
  int best_pairs = 8;
  double best = 1e30;
  for (int r = 2; r <= 16; ++r) {
    const int blocks = (pairs + r - 1) / r;
    const double bytes = 4.0 * r * K + (norm ? 4.0 * min(T, 16) * K + 2.0 * K : 2.0 * T * K);
    const double cost = double((blocks * token_tiles + 255) / 256) * bytes;
    if (cost <= best) { best = cost; best_pairs = r; }
  }
  return best_pairs;
}

template <int EPI, bool NORM>
static int fused_tokens(hipStream_t s, const FusedArgs& a, int blocks, int splits) {
  if constexpr (EPI == kEpiSilu) {   // up to 16 tokens: a block may own up to 24 inner columns (three tiles)
    if (a.rows_per_block > 16) return launch_fused<1, EPI, NORM, 3>(s, a, blocks, splits);
  }
  if constexpr (NORM) {   // tiles of 16 tokens, each a block of its own
    if constexpr (EPI == kEpiRope) {
      if (a.rows_per_block <= 8) return launch_fused<1, EPI, true, 1>(s, a, blocks, splits);   // one gathered tile
    }
    return launch_fused<1, EPI, true>(s, a, blocks, splits);
  } else {
    if (EPI == kEpiRope && a.rows_per_block <= 8) {
      if constexpr (EPI == kEpiRope) {
        if (a.T <= 16) return launch_fused<1, EPI, false, 1>(s, a, blocks, splits);
        if (a.T <= 32) return launch_fused<2, EPI, false, 1>(s, a, blocks, splits);
        return launch_fused<4, EPI, false, 1>(s, a, blocks, splits);
      }
    }
    if (a.T <= 16) return launch_fused<1, EPI, false>(s, a, blocks, splits);
    // More than 32 tokens: tiles of 32 along the grid's z while the matrix is small.  A block that takes all 64
    // reads twice the activations for the same weight rows (64 tokens, 896 x 896: 4.9 us against 3.9; 896 x 4,864
    // the same either way), tiles of 16 read the weights four times (4.4 and 9.1 us), and a large matrix is read
    // once whatever that costs in activations (4,608 x 3,584: 20 us with all 64 tokens a block, 28 in tiles of 32).
    if (a.T <= 32 || size_t(a.N) * a.K <= (size_t(2) << 20)) return launch_fused<2, EPI, false>(s, a, blocks, splits);
    return launch_fused<4, EPI, false>(s, a, blocks, splits);
  }
}

// Inner columns a block of the gated product owns.  A CU pulls its blocks' rows at about the same rate however
// many blocks it holds, so the matrix is cut for the CU that gets the most: bytes a block asks for (its gate and
// up rows, and the activations, which every block reads whole) times blocks per CU, rounded up.  4,864 inner
// columns: 256 blocks of 19 instead of 304 of 16, of which 48 CUs held two.  More than 16 columns (three tiles)
// only where a block takes one tile of tokens (up to 16 tokens, or the norm prologue).
static int silu_rows_per_block(int T, int I, int K, bool norm) {
  const int most = (T <= 16 || norm) ? 24 : 16;
  const int token_tiles = norm ? (T + 15) / 16 : 1;
  int best_rows = 16;
  double best = 1e30;
  for (int r = 4; r <= most; ++r) {
    const int blocks = (I + r - 1) / r;
    const double bytes = 4.0 * r * K + (norm ? 4.0 * min(T, 16) * K + 2.0 * K : 2.0 * T * K);
    const double cost = double((blocks * token_tiles + 255) / 256) * bytes;
    if (cost <= best) { best = cost; best_rows = r; }
  }
  return best_rows;
}

template <int EPI>
static int fused_norm(hipStream_t s, const FusedArgs& a, bool norm, int blocks, int splits) {
  return norm ? fused_tokens<EPI, true>(s, a, blocks, splits) : fused_tokens<EPI, false>(s, a, blocks, splits);
}

// Whether the fused kernels take this shape: K in 16-byte rows, T <= 64.
static bool fused_shape_ok(int T, int K, bool norm) {
  (void)norm;
  return T >= 1 && T <= 64 && K % 8 == 0;
}

}  // namespace sprout

using namespace sprout;

extern "C" int sp_gemm_decode(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w,
                              float eps, const void* w, int bias_dtype, const void* bias, int mode, void* out, int T,
                              int N, int K);

namespace sprout {
int gemm_bf16_tiled_silu(hipStream_t s, const void* x, const void* w, void* out, int T, int I, int K);
bool gemm_pipe_takes(int T, int N, int K);
bool gemm_pipe_rope_takes(int T, int N, int K, int hd);
int gemm_bf16_pipe_rope(hipStream_t s, const void* x, const void* w, int bias_dtype, const void* bias, void* q_out,
                        const int32_t* positions, const float* inv_freq, const int32_t* slot_mapping, void* k_pool,
                        void* v_pool, int T, int K, int nq, int nkv, int hd, int page_size, const float* table);
}

extern "C" int sp_fused_supported(int kind, int T, int N, int K, int hd, int rotary_dim, int norm, int variant) {
  if (variant != 0) return 0;   // the one pairing (halves) and the one activation (SiLU) these kernels have
  if (kind == kEpiSilu && T > 64) return !norm && K % 8 == 0 && N % 2 == 0;   // the tiled kernel's gated epilogue
  if (kind == kEpiRope && T > 64) return !norm && rotary_dim == hd && gemm_pipe_rope_takes(T, N, K, hd);   // and its rotating one
  if (!fused_shape_ok(T, K, norm != 0)) return 0;
  if (kind == kEpiRope) return hd % 16 == 0 && (rotary_dim == hd || rotary_dim == 0) && N % hd == 0;
  if (kind == kEpiSilu) return N % 32 == 0;
  return kind == kEpiStore || kind == kEpiAccumulate || kind == kEpiStoreF32;
}

// Whether the norm prologue is faster than a norm kernel of its own before the product.  Every block reads
// its 16 tokens' rows of the float32 residual beside its weight rows, which costs more the wider the rows are:
// measured at 8 tokens, QKV product with prologue against norm kernel + product: 7.0 against 7.9 us at a
// width of 896, 11.6 against 9.4 at 1536, 22.2 against 16.2 at 3584; the gated product alike.  With more than
// 16 tokens every tile of tokens reads the weights again: that pays while all the blocks run at once (1,152 rows
// x 896 at 64 tokens: 8.6 us against 8.7 + 2.4 for the norm), not beyond (9,728 x 896: 21.2 against 8.5 + 2.4).
extern "C" int sp_fused_norm_pays(int T, int N, int K) {
  if (!fused_shape_ok(T, K, true) || K > 1024) return 0;
  return T <= 16 || (N / 16) * ((T + 15) / 16) <= 512;
}

namespace sprout {
int gemm_decode_plain(hipStream_t s, const void* x, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                      int T, int N, int K) {
  return sp_gemm_decode((void*)s, x, nullptr, 0, nullptr, 0.f, w, bias_dtype, bias, mode, out, T, N, K);
}
}  // namespace sprout

// Plain product through the K-splitting kernel: out = x . w^T (+ bias), modes as sp_gemm.
// With residual != null the activations are rmsnorm(residual) * norm_w instead of x.
extern "C" int sp_gemm_decode(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w,
                              float eps, const void* w, int bias_dtype, const void* bias, int mode, void* out, int T,
                              int N, int K) {
  SP_REQUIRE(mode >= 0 && mode <= 2, "sp_gemm_decode: unknown mode %d", mode);
  SP_REQUIRE(fused_shape_ok(T, K, residual != nullptr), "sp_gemm_decode: shape T=%d K=%d is not taken", T, K);
  SP_REQUIRE((x || residual) && w && out && N > 0, "sp_gemm_decode: null operand");
  FusedArgs a = {};
  a.x = (const uint16_t*)x; a.residual = residual; a.norm_w = norm_w; a.norm_w_bf16 = norm_w_dtype == kBF16; a.eps = eps;
  a.w = (const uint16_t*)w; a.bias = bias; a.bias_bf16 = bias_dtype == kBF16; a.out = out;
  a.T = T; a.N = N; a.K = K;
  const int blocks = (N + 31) / 32;
  int splits = 1;
  a.k_per_split = (K + 63) / 64 * 64;
  if (mode == kEpiAccumulate && !residual) {
    // A CU pulls its blocks' weight rows at about the same rate however many blocks it holds, so the split of K
    // is chosen for the CU that gets the most: blocks per CU (rounded up) x bytes per block, plus the float
    // atomics of the split (measured 2.7 us per million added floats), both in microseconds.  (8 tokens, against
    // a fixed aim of 768 blocks: 18,944 x 3,584 36 -> 31 us, 27,648 x 5,120 64 -> 55 us, 4,864 x 896 6.0 -> 5.5 us.)
    float best = 1e30f;
    for (int sp = 1; sp <= min(64, max(1, K / 256)); ++sp) {
      const int k_per = ((K + sp - 1) / sp + 63) / 64 * 64, real = (K + k_per - 1) / k_per;
      const float per_cu = float((blocks * real + 255) / 256) * 32.f * float(k_per) * 2.f;   // bytes
      const float cost = per_cu / 20e3f + 2.7e-6f * float(T) * float(N) * float(real) + (real > 1 ? 0.3f : 0.f);
      if (cost < best) { best = cost; splits = real; a.k_per_split = k_per; }
    }
  }
  hipStream_t s = (hipStream_t)stream;
  if (mode == kEpiStore) return fused_norm<kEpiStore>(s, a, residual != nullptr, blocks, splits);
  if (mode == kEpiAccumulate) return fused_norm<kEpiAccumulate>(s, a, residual != nullptr, blocks, splits);
  return fused_norm<kEpiStoreF32>(s, a, residual != nullptr, blocks, splits);
}

// q/k/v projection with bias, rotation and cache write.  w is [(nq + 2 nkv) * hd, K] (q, k, v rows).
// q_out: [T, nq * hd] bfloat16.  Activations: x, or rmsnorm(residual) * norm_w if residual != null.
extern "C" int sp_qkv_rope_cache(void* stream, const void* x, const float* residual, int norm_w_dtype,
                                 const void* norm_w, float eps, const void* w, int bias_dtype, const void* bias,
                                 void* q_out, const int32_t* positions, const float* inv_freq, int rotary_dim,
                                 const int32_t* slot_mapping, void* k_pool, void* v_pool, int T, int K, int nq,
                                 int nkv, int hd, int page_size, const float* cos_sin, int pairing) {
  const int N = (nq + 2 * nkv) * hd;
  SP_REQUIRE(pairing == 0, "sp_qkv_rope_cache: no kernel for pairing %d (0 = halves of the rotated dimensions)", pairing);
  SP_REQUIRE(sp_fused_supported(kEpiRope, T, N, K, hd, rotary_dim, residual != nullptr, pairing),
             "sp_qkv_rope_cache: shape T=%d K=%d hd=%d rotary=%d is not taken", T, K, hd, rotary_dim);
  SP_REQUIRE((x || residual) && w && q_out && positions && inv_freq && slot_mapping && k_pool && v_pool,
             "sp_qkv_rope_cache: null operand");
  if (T > 64)   // many tokens: the pipelined tiled product with the rotation as its epilogue
    return gemm_bf16_pipe_rope((hipStream_t)stream, x, w, bias_dtype, bias, q_out, positions, inv_freq, slot_mapping, k_pool,
                               v_pool, T, K, nq, nkv, hd, page_size, cos_sin);
  FusedArgs a = {};
  a.x = (const uint16_t*)x; a.residual = residual; a.norm_w = norm_w; a.norm_w_bf16 = norm_w_dtype == kBF16; a.eps = eps;
  a.w = (const uint16_t*)w; a.bias = bias; a.bias_bf16 = bias_dtype == kBF16; a.out = q_out;
  a.T = T; a.N = N; a.K = K; a.k_per_split = (K + 63) / 64 * 64; a.partner = hd / 2;
  a.positions = positions; a.inv_freq = inv_freq; a.slot_mapping = slot_mapping;
  a.k_pool = (uint16_t*)k_pool; a.v_pool = (uint16_t*)v_pool;
  a.nq = nq; a.nkv = nkv; a.hd = hd; a.page_size = page_size; a.rotary_dim = rotary_dim;
  a.page_shift = -1;
  if (page_size > 0 && (page_size & (page_size - 1)) == 0)
    for (a.page_shift = 0; (1 << a.page_shift) < page_size;) ++a.page_shift;
  a.rows_per_block = rope_pairs_per_block(T, N, K, residual != nullptr);
  const int blocks = (N / 2 + a.rows_per_block - 1) / a.rows_per_block;
  return fused_norm<kEpiRope>((hipStream_t)stream, a, residual != nullptr, blocks, 1);
}

// out[T, I] = silu(x . w_gate^T) * (x . w_up^T) with w = [gate rows; up rows] of [2 I, K].
extern "C" int sp_gate_up_silu(void* stream, const void* x, const float* residual, int norm_w_dtype,
                               const void* norm_w, float eps, const void* w, void* out, int T, int I, int K,
                               int activation) {
  SP_REQUIRE(activation == 0, "sp_gate_up_silu: no kernel for activation %d (0 = SiLU)", activation);
  SP_REQUIRE(sp_fused_supported(kEpiSilu, T, 2 * I, K, 0, 0, residual != nullptr, activation),
             "sp_gate_up_silu: shape T=%d I=%d K=%d is not taken", T, I, K);
  SP_REQUIRE((x || residual) && w && out, "sp_gate_up_silu: null operand");
  // Many tokens, or a few with whole steps of 64 along K: the tiled kernels stream the weights better.  From 17
  // tokens on always; from 9 on where the matrix is large, from 5 on where it is very large (a step of the
  // whole model at 8 tokens, fused against tiled: 2 x 18,944 x 3,584 3.77 against 3.84 ms, at 16 tokens 4.35 against
  // 4.30; 2 x 27,648 x 5,120 at 8 tokens 14.82 against 14.70, at 16 17.17 against 16.30; 2 x 8,960 x 1,536 at 8
  // tokens 15.5 us fused against 16.7).
  const size_t weights = size_t(2) * I * K;
  const int fused_up_to = weights >= (size_t(200) << 20) ? 4 : weights >= (size_t(64) << 20) ? 8 : 16;
  if (T > 64 || (T > fused_up_to && !residual && gemm_pipe_takes(T, 2 * I, K)))
    return gemm_bf16_tiled_silu((hipStream_t)stream, x, w, out, T, I, K);
  FusedArgs a = {};
  a.x = (const uint16_t*)x; a.residual = residual; a.norm_w = norm_w; a.norm_w_bf16 = norm_w_dtype == kBF16; a.eps = eps;
  a.w = (const uint16_t*)w; a.out = out;
  a.T = T; a.N = 2 * I; a.K = K; a.k_per_split = (K + 63) / 64 * 64; a.partner = I;
  a.rows_per_block = silu_rows_per_block(T, I, K, residual != nullptr);
  return fused_norm<kEpiSilu>((hipStream_t)stream, a, residual != nullptr, (I + a.rows_per_block - 1) / a.rows_per_block, 1);
}
