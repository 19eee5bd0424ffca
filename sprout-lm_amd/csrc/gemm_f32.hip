// Tiled float32 product for more than a handful of tokens: out[T, N] (float32) = or += x[T, K] . w[N, K]^T with
// float32 operands, on v_mfma_f32_32x32x2_f32 (true 32-bit products and sums; no reduced-precision mode).  The
// kernel is the pipelined tiled product of gemm_pipe.h with float operands; K must be a multiple of 32 (rows of
// whole 128-byte slices).  Everything else (few tokens, other K, mixed operand types) stays on the FMA kernels.
#include "gemm_pipe.h"

namespace sprout {

namespace {

struct F32Shape { int bm, bn; float cost; };   // cost: time of a block per unit of area, against the largest shape
constexpr F32Shape kShapes[4] = {{256, 128, 1.0f}, {128, 128, 1.05f}, {64, 128, 1.12f}, {64, 64, 1.25f}};

// The matrix cores bound this product, so a launch takes as long as the CU with the most tile area: the shape
// with the least (blocks on the fullest CU) x (tile area) x (what a smaller tile loses to its fetches).
int choose_shape(int T, int N) {
  int best = 0;
  float best_cost = 0.f;
  for (int i = 0; i < 4; ++i) {
    const long blocks = long((T + kShapes[i].bm - 1) / kShapes[i].bm) * ((N + kShapes[i].bn - 1) / kShapes[i].bn);
    const float cost = float((blocks + 255) / 256) * kShapes[i].bm * kShapes[i].bn * kShapes[i].cost;
    if (i == 0 || cost < best_cost) { best = i; best_cost = cost; }
  }
  return best;
}

template <int WM, int WN, int WAVES_M, int WAVES_N, int STAGES, typename TB>
int launch_f32(hipStream_t s, const float* x, const float* w, const void* bias, int mode, float* out, int T, int N, int K) {
  if (mode == kAccumulate)
    return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kAccumulate, TB, float>(s, 1, x, w, (const TB*)bias, out, T, N, K, K);
  return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kStoreF32, TB, float>(s, 1, x, w, (const TB*)bias, out, T, N, K, K);
}

template <typename TB>
int launch_shape(hipStream_t s, const float* x, const float* w, const void* bias, int mode, float* out, int T, int N, int K) {
  switch (choose_shape(T, N)) {
    case 0: return launch_f32<2, 2, 4, 2, 3, TB>(s, x, w, bias, mode, out, T, N, K);
    case 1: return launch_f32<1, 2, 4, 2, 4, TB>(s, x, w, bias, mode, out, T, N, K);
    case 2: return launch_f32<1, 2, 2, 2, 3, TB>(s, x, w, bias, mode, out, T, N, K);
    default: return launch_f32<1, 1, 2, 2, 4, TB>(s, x, w, bias, mode, out, T, N, K);
  }
}

}  // namespace

bool gemm_f32_takes(int T, int N, int K, const void* a, const void* w, const void* out) {
  return T > 16 && K % 32 == 0 && K >= 32 && int64_t(K) * 4 * 256 < (int64_t(1) << 32) &&
         (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
}

// mode: kAccumulate (out += ...) or anything else (out = ...); out is float32 either way.
int gemm_f32(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out, int T,
             int N, int K) {
  if (bias && bias_dtype == kBF16)
    return launch_shape<bf16_t>(s, (const float*)a, (const float*)w, bias, mode, (float*)out, T, N, K);
  return launch_shape<float>(s, (const float*)a, (const float*)w, bias, mode, (float*)out, T, N, K);
}

}  // namespace sprout

// ---------------------------------------------------------------------------------------------- few tokens
// Up to 16 tokens (decoding): the weights are read once and the product is bound by how many bytes the chip has
// on their way, so the work is cut fine: a block is four waves that share K in quarters and take RT tiles of 16
// weight rows; in accumulate mode K is also split over blocks (float atomics) where the rows alone give too few.
//   D[weight row, token] += W[row, k] . X[token, k]     v_mfma_f32_16x16x4_f32, A = weights, B = activations
// A lane loads 16 bytes of a weight row (4 numbers that feed 4 successive MFMAs) and 16 bytes of a token's
// activations, which serve every row tile of the wave; no sum crosses lanes.  The four waves' sums meet in LDS
// in a fixed order.  K must be a multiple of 4.
namespace sprout {

namespace {

typedef float floatx4_t __attribute__((ext_vector_type(4)));

// MODE kSilu: w holds N gate rows, then N up rows; the block's RT tiles are RT / 2 tiles of gate rows and the
// matching tiles of up rows, and out[t, n] = silu(gate) * up (float32 [T, N]).
template <int RT, int MODE, typename TB>   // MODE: kStoreF32, kAccumulate or kSilu
__global__ __launch_bounds__(256) void gemm_f32_skinny_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                              const TB* __restrict__ bias, float* __restrict__ out,
                                                              int T, int N, int K, int steps_per_block) {
  __shared__ float sums[4][RT][64][4];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  const int n0 = blockIdx.x * 16 * (MODE == kSilu ? RT / 2 : RT);
  const int total_steps = (K + 15) / 16;
  const int first = blockIdx.y * steps_per_block, last = min(total_steps, first + steps_per_block);
  // this wave's steps of the block's: a contiguous quarter
  const int mine = (last - first + 3) / 4;
  const int s0 = first + wave * mine, s1 = min(last, s0 + mine);

  const float* wrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = MODE == kSilu ? min(n0 + 16 * (rt / 2) + lr, N - 1) + (rt & 1) * N : min(n0 + 16 * rt + lr, N - 1);
    wrow[rt] = w + size_t(row) * K + 4 * lj;
  }
  const float* xrow = x + size_t(min(lr, T - 1)) * K + 4 * lj;
  const bool token = lr < T;

  floatx4_t acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  constexpr int U = RT <= 2 ? 8 : 4;      // steps requested together: what a wave has on its way
  for (int s = s0; s < s1; s += U) {
    float4 wv[U][RT], xv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = 16 * (s + u);
      const bool in = s + u < s1 && k + 4 * lj < K;
      xv[u] = (in && token) ? *reinterpret_cast<const float4*>(xrow + k) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        wv[u][rt] = in ? *reinterpret_cast<const float4*>(wrow[rt] + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].x, xv[u].x, acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].y, xv[u].y, acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].z, xv[u].z, acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].w, xv[u].w, acc[rt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
    *reinterpret_cast<float4*>(&sums[wave][rt][lane][0]) = make_float4(acc[rt][0], acc[rt][1], acc[rt][2], acc[rt][3]);
  __syncthreads();
  // thread (rt, lane) of the first RT waves' worth of threads joins the four waves: element e is
  // out[token lane % 16][n0 + 16 rt + 4 (lane / 16) + e]
  if (MODE == kSilu) {
    for (int i = threadIdx.x; i < RT / 2 * 64; i += 256) {
      const int pair = i >> 6, l = i & 63, t = l & 15, n = n0 + 16 * pair + 4 * (l >> 4);
      if (t >= T || n >= N) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (n + e >= N) break;
        const int a = 2 * pair, b = 2 * pair + 1;
        const float gate = ((sums[0][a][l][e] + sums[1][a][l][e]) + sums[2][a][l][e]) + sums[3][a][l][e];
        const float up = ((sums[0][b][l][e] + sums[1][b][l][e]) + sums[2][b][l][e]) + sums[3][b][l][e];
        out[size_t(t) * N + n + e] = gate / (1.0f + expf(-gate)) * up;
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < RT * 64; i += 256) {
    const int rt = i >> 6, l = i & 63, t = l & 15, n = n0 + 16 * rt + 4 * (l >> 4);
    if (t >= T || n >= N) continue;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = ((sums[0][rt][l][e] + sums[1][rt][l][e]) + sums[2][rt][l][e]) + sums[3][rt][l][e];
    float* dst = out + size_t(t) * N + n;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (n + e >= N) break;
      float r = v[e];
      if (bias && blockIdx.y == 0) r += to_float(bias[n + e]);
      if (MODE == kAccumulate) {
        if (gridDim.y > 1) unsafeAtomicAdd(dst + e, r);
        else dst[e] += r;
      } else {
        dst[e] = r;
      }
    }
  }
}

template <int RT, typename TB>
int launch_skinny(hipStream_t s, const float* x, const float* w, const void* bias, int mode, float* out, int T, int N, int K) {
  const int blocks_n = (N + 16 * RT - 1) / (16 * RT), steps = (K + 15) / 16;
  int splits = 1;
  if (mode == kAccumulate && blocks_n < 256) {
    // rows alone give too few blocks: K is shared out too, while every wave keeps 8 steps or more
    splits = max(1, min((512 + blocks_n - 1) / blocks_n, steps / 32));
  }
  const int per_block = (steps + splits - 1) / splits;
  splits = (steps + per_block - 1) / per_block;
  dim3 grid(blocks_n, splits);
  if (mode == kAccumulate)
    gemm_f32_skinny_kernel<RT, kAccumulate, TB><<<grid, 256, 0, s>>>(x, w, (const TB*)bias, out, T, N, K, per_block);
  else
    gemm_f32_skinny_kernel<RT, kStoreF32, TB><<<grid, 256, 0, s>>>(x, w, (const TB*)bias, out, T, N, K, per_block);
  return check_launch("sp_gemm (float32, few tokens)");
}

template <typename TB>
int skinny_shape(hipStream_t s, const float* x, const float* w, const void* bias, int mode, float* out, int T, int N, int K) {
  const int tiles = (N + 15) / 16;
  if (tiles >= 4096) return launch_skinny<4, TB>(s, x, w, bias, mode, out, T, N, K);
  if (tiles >= 1024) return launch_skinny<2, TB>(s, x, w, bias, mode, out, T, N, K);
  return launch_skinny<1, TB>(s, x, w, bias, mode, out, T, N, K);
}

}  // namespace

// out[T, I] = silu(x . w[:I]^T) * (x . w[I:]^T) for up to 16 tokens, float32 throughout.
int gemm_f32_gated(hipStream_t s, const float* x, const float* w, float* out, int T, int I, int K) {
  const int pairs = (I + 15) / 16;
  if (pairs >= 2048) {
    gemm_f32_skinny_kernel<4, kSilu, float><<<dim3((pairs + 1) / 2, 1), 256, 0, s>>>(x, w, nullptr, out, T, I, K, (K + 15) / 16);
  } else {
    gemm_f32_skinny_kernel<2, kSilu, float><<<dim3(pairs, 1), 256, 0, s>>>(x, w, nullptr, out, T, I, K, (K + 15) / 16);
  }
  return check_launch("sp_gate_up_silu (float32, few tokens)");
}

bool gemm_f32_skinny_takes(int T, int N, int K, const void* a, const void* w) {
  return T >= 1 && T <= 16 && K % 4 == 0 && K >= 64 &&
         (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) % 16 == 0;
}

int gemm_f32_skinny(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                    int T, int N, int K) {
  if (bias && bias_dtype == kBF16)
    return skinny_shape<bf16_t>(s, (const float*)a, (const float*)w, bias, mode, (float*)out, T, N, K);
  return skinny_shape<float>(s, (const float*)a, (const float*)w, bias, mode, (float*)out, T, N, K);
}

}  // namespace sprout

using namespace sprout;

// Whether sp_gate_up_silu_f32 takes T tokens by 2 I rows of K.
extern "C" int sp_gate_up_silu_f32_takes(int T, int I, int K) { return T >= 1 && T <= 16 && I >= 1 && K % 4 == 0 && K >= 64; }

// out[T, I] (float32) = act(x . w[:I]^T) * (x . w[I:]^T), x float32 [T, K], w float32 [2 I, K], up to 16 tokens:
// the gated product of a decode step on the float32 path, in one kernel.
extern "C" int sp_gate_up_silu_f32(void* stream, const float* x, const float* w, float* out, int T, int I, int K,
                                   int activation) {
  SP_REQUIRE(activation == 0, "sp_gate_up_silu_f32: no kernel for activation %d (0 = SiLU)", activation);
  SP_REQUIRE(sp_gate_up_silu_f32_takes(T, I, K), "sp_gate_up_silu_f32: shape T=%d I=%d K=%d is not taken", T, I, K);
  SP_REQUIRE(x && w && out && (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) % 16 == 0,
             "sp_gate_up_silu_f32: operands must be given and 16-byte aligned");
  return gemm_f32_gated((hipStream_t)stream, x, w, out, T, I, K);
}
