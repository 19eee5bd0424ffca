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
// NORM: the activations are rmsnorm(x) * norm_w of the float32 residual x, computed here ((x * scale) * w, the
// very numbers the norm kernel stores): every block sums the squares of its tokens' rows first.
// MODE kSilu: w holds N gate rows, then N up rows; the block's RT tiles are RT / 2 tiles of gate rows and the
// matching tiles of up rows (RT = 1: one tile of 8 gate rows, tile rows 0-7, and the matching 8 up rows, 8-15), and
// out[t, n] = silu(gate) * up (float32 [T, N]).
// MODE kRope: the rows of w are q, k and v heads of size hd (a multiple of 16); a block's tile is 8 dimensions of
// a head's first half (tile rows 0-7) and their rotation partners half a head further on (rows 8-15): twice the
// blocks of whole tiles of 16, and these products live on how many blocks stream.  Bias, rotation of q and k
// heads by positions * inv_freq (angle, sine and cosine in float64 where inv_freq_tail is given), q to out
// [T, nq * hd], k and v into the paged pools.
namespace sprout {

namespace {

typedef float floatx4_t __attribute__((ext_vector_type(4)));

struct SkinnyExtra {
  const float* norm_w;          // NORM
  float eps;
  // kRope
  const int32_t* positions;
  const float* inv_freq;
  const float* inv_freq_tail;   // may be null
  const int32_t* slot_mapping;
  float* k_pool;                // [page][kv head][slot][dim]
  float* v_pool;                // [page][kv head][dim][slot]
  int nq, nkv, hd, page_size, num_pages;
};

template <int RT, int MODE, typename TB, bool NORM, int WAVES = 4>   // MODE: kStoreF32, kAccumulate, kSilu or kRope
__global__ __launch_bounds__(64 * WAVES) void gemm_f32_skinny_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                              const TB* __restrict__ bias, float* __restrict__ out,
                                                              int T, int N, int K, int steps_per_block, SkinnyExtra extra) {
  static_assert(WAVES == 4 || WAVES == 8, "four or eight waves share K");
  __shared__ float sums[WAVES][RT][64][4];
  __shared__ float row_scale[16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  const int total_steps = (K + 15) / 16;
  const int first = blockIdx.y * steps_per_block, last = min(total_steps, first + steps_per_block);
  // this wave's steps of the block's: a contiguous share
  const int mine = (last - first + WAVES - 1) / WAVES;
  const int s0 = first + wave * mine, s1 = min(last, s0 + mine);

  int n0 = MODE == kSilu && RT == 1 ? blockIdx.x * 8 : blockIdx.x * 16 * (MODE == kSilu ? RT / 2 : RT);
  const float* wrow[RT];
  if (MODE == kRope) {
    static_assert(MODE != kRope || RT == 1, "a block of the rotating product is one tile: 8 dimensions and their partners");
    const int per_head = extra.hd / 16, head = blockIdx.x / per_head, u = blockIdx.x % per_head;
    n0 = head * extra.hd + 8 * u;
    wrow[0] = w + size_t(n0 + (lr & 7) + (lr >> 3) * (extra.hd / 2)) * K + 4 * lj;
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      int row;
      if (MODE == kSilu && RT == 1) row = min(n0 + (lr & 7), N - 1) + (lr >> 3) * N;
      else if (MODE == kSilu) row = min(n0 + 16 * (rt / 2) + lr, N - 1) + (rt & 1) * N;
      else row = min(n0 + 16 * rt + lr, N - 1);
      wrow[rt] = w + size_t(row) * K + 4 * lj;
    }
  }
  const float* xrow = x + size_t(min(lr, T - 1)) * K + 4 * lj;
  const bool token = lr < T;

  constexpr int U = RT <= 2 ? 8 : 4;      // steps requested together: what a wave has on its way
  float4 wv[U][RT], xv[U], nv[U];
  auto request = [&](int s) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = 16 * (s + u);
      const bool in = s + u < s1 && k + 4 * lj < K;
      xv[u] = (in && token) ? *reinterpret_cast<const float4*>(xrow + k) : make_float4(0.f, 0.f, 0.f, 0.f);
      if (NORM) nv[u] = in ? *reinterpret_cast<const float4*>(extra.norm_w + k + 4 * lj) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        wv[u][rt] = in ? *reinterpret_cast<const float4*>(wrow[rt] + k) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };
  // NORM: thread (token threadIdx.x / P, part threadIdx.x % P) sums its share of the squares of the token's row,
  // 8 loads at a time.  The first 8 are asked for before the weights (they come from the
  // caches, and what returns from memory returns in the order asked for), the weights before anything is summed:
  // they are on their way meanwhile, and the rest of a longer row queues behind them.
  float scale = 1.f;
  if (NORM) {
    constexpr int P = 4 * WAVES, NB = 8;
    const int t = threadIdx.x / P, part = threadIdx.x % P;
    const float* row = x + size_t(min(t, T - 1)) * K;
    float4 part_x[NB];
    auto ask = [&](int k0) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int k = k0 + j * 4 * P;
        part_x[j] = (t < T && k < K) ? *reinterpret_cast<const float4*>(row + k) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    };
    float sum = 0.f;
    auto add = [&]() {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const float4 v = part_x[j];
        sum = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, sum))));
      }
    };
    ask(4 * part);
    request(s0);
    add();
    for (int k0 = 4 * part + NB * 4 * P; k0 < K; k0 += NB * 4 * P) {
      ask(k0);
      add();
    }
#pragma unroll
    for (int o = P / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
    if (part == 0) row_scale[t] = 1.0f / sqrtf(sum / float(K) + extra.eps);
    __syncthreads();
    scale = token ? row_scale[lr] : 0.f;      // lanes past the last token multiply zeros
  } else {
    request(s0);
  }

  floatx4_t acc[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  for (int s = s0; s < s1; s += U) {
    if (s != s0) request(s);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (s + u >= s1) break;      // the same for the whole wave
      if (NORM)
        xv[u] = make_float4((xv[u].x * scale) * nv[u].x, (xv[u].y * scale) * nv[u].y, (xv[u].z * scale) * nv[u].z,
                            (xv[u].w * scale) * nv[u].w);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].x, xv[u].x, acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].y, xv[u].y, acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].z, xv[u].z, acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[u][rt].w, xv[u].w, acc[rt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
    *reinterpret_cast<float4*>(&sums[wave][rt][lane][0]) = make_float4(acc[rt][0], acc[rt][1], acc[rt][2], acc[rt][3]);
  __syncthreads();
  // Element e of lane l of tile rt is out[token l % 16][tile row 4 (l / 16) + e]; the waves are joined in order.
  auto joined = [&](int rt, int l, int e) {
    float sum = sums[0][rt][l][e];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += sums[w][rt][l][e];
    return sum;
  };
  if (MODE == kRope) {
    // thread (token t, row r < 8): tile row r is element r % 4 of lane t + 16 (r / 4), its partner row r + 8 lies
    // two quarters of the wave further on
    if (threadIdx.x >= 128) return;
    const int t = threadIdx.x & 15, r = threadIdx.x >> 4;
    if (t >= T) return;
    const int hd = extra.hd, half = hd / 2;
    const int head = n0 / hd, d = n0 % hd + r;                       // the dimension of the first half
    float a = joined(0, t + 16 * (r >> 2), r & 3), b = joined(0, t + 16 * (r >> 2) + 32, r & 3);
    if (bias) { a += to_float(bias[head * hd + d]); b += to_float(bias[head * hd + d + half]); }
    if (head < extra.nq + extra.nkv) {
      float sn, cs;
      if (extra.inv_freq_tail) {
        double sn64, cs64;
        sincos(double(extra.positions[t]) * (double(extra.inv_freq[d]) + double(extra.inv_freq_tail[d])), &sn64, &cs64);
        sn = float(sn64);
        cs = float(cs64);
      } else {
        sincosf(float(extra.positions[t]) * extra.inv_freq[d], &sn, &cs);
      }
      const float ra = a * cs - b * sn, rb = b * cs + a * sn;
      a = ra;
      b = rb;
    }
    if (head < extra.nq) {
      float* q = out + size_t(t) * (size_t(extra.nq) * hd) + head * hd + d;
      q[0] = a;
      q[half] = b;
      return;
    }
    const int slot = extra.slot_mapping[t];
    if (slot < 0) return;
    const int page = slot / extra.page_size, off = slot % extra.page_size;
    if (page >= extra.num_pages) return;                       // a bad slot must not become a wild address
    if (head < extra.nq + extra.nkv) {
      float* k = extra.k_pool + ((size_t(page) * extra.nkv + (head - extra.nq)) * extra.page_size + off) * hd + d;
      k[0] = a;
      k[half] = b;
    } else {
      float* v = extra.v_pool + ((size_t(page) * extra.nkv + (head - extra.nq - extra.nkv)) * hd + d) * extra.page_size + off;
      v[0] = a;
      v[size_t(half) * extra.page_size] = b;
    }
    return;
  }
  if (MODE == kSilu && RT == 1) {
    if (threadIdx.x >= 128) return;
    const int t = threadIdx.x & 15, r = threadIdx.x >> 4, n = n0 + r;
    if (t >= T || n >= N) return;
    const float gate = joined(0, t + 16 * (r >> 2), r & 3), up = joined(0, t + 16 * (r >> 2) + 32, r & 3);
    out[size_t(t) * N + n] = gate / (1.0f + expf(-gate)) * up;
    return;
  }
  if (MODE == kSilu) {
    for (int i = threadIdx.x; i < RT / 2 * 64; i += 64 * WAVES) {
      const int pair = i >> 6, l = i & 63, t = l & 15, n = n0 + 16 * pair + 4 * (l >> 4);
      if (t >= T || n >= N) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (n + e >= N) break;
        const float gate = joined(2 * pair, l, e), up = joined(2 * pair + 1, l, e);
        out[size_t(t) * N + n + e] = gate / (1.0f + expf(-gate)) * up;
      }
    }
    return;
  }
  // thread -> (token, row of the block): neighbouring threads take neighbouring rows of one token, so that a wave
  // writes or adds runs of 16 RT numbers (atomics scattered one number at a time take several times longer)
  for (int i = threadIdx.x; i < RT * 256; i += 64 * WAVES) {
    const int t = i / (16 * RT), row = i % (16 * RT), n = n0 + row;
    if (t >= T || n >= N) continue;
    float r = joined(row >> 4, t + 16 * ((row & 15) >> 2), row & 3);
    if (bias && blockIdx.y == 0) r += to_float(bias[n]);
    float* dst = out + size_t(t) * N + n;
    if (MODE == kAccumulate) {
      if (gridDim.y > 1) unsafeAtomicAdd(dst, r);
      else *dst += r;
    } else {
      *dst = r;
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
    gemm_f32_skinny_kernel<RT, kAccumulate, TB, false><<<grid, 256, 0, s>>>(x, w, (const TB*)bias, out, T, N, K, per_block, SkinnyExtra{});
  else
    gemm_f32_skinny_kernel<RT, kStoreF32, TB, false><<<grid, 256, 0, s>>>(x, w, (const TB*)bias, out, T, N, K, per_block, SkinnyExtra{});
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

// out[T, I] = silu(a . w[:I]^T) * (a . w[I:]^T) for up to 16 tokens, float32 throughout; a = x, or
// rmsnorm(x) * norm_w where norm_w is given.
int gemm_f32_gated(hipStream_t s, const float* x, const float* norm_w, float eps, const float* w, float* out, int T, int I, int K) {
  const int pairs = (I + 15) / 16, steps = (K + 15) / 16;
  SkinnyExtra extra = {};
  extra.norm_w = norm_w;
  extra.eps = eps;
#define SP_GATED(RT, NORM, BLOCKS) \
  gemm_f32_skinny_kernel<RT, kSilu, float, NORM><<<dim3(BLOCKS, 1), 256, 0, s>>>(x, w, nullptr, out, T, I, K, steps, extra)
  if (pairs >= 2048) {
    if (norm_w) SP_GATED(4, true, (pairs + 1) / 2); else SP_GATED(4, false, (pairs + 1) / 2);
  } else if (pairs >= 512) {
    if (norm_w) SP_GATED(2, true, pairs); else SP_GATED(2, false, pairs);
  } else {
    // few rows: tiles of 8 gate rows and their 8 up rows, twice the blocks
    if (norm_w) SP_GATED(1, true, (I + 7) / 8); else SP_GATED(1, false, (I + 7) / 8);
  }
#undef SP_GATED
  return check_launch("sp_gate_up_silu_f32");
}

template <typename TB, int WAVES>
static int launch_qkv_waves(hipStream_t s, const float* x, const float* w, const void* bias, float* q_out, int T, int K,
                            const SkinnyExtra& extra, int N, int blocks, int steps) {
  if (extra.norm_w)
    gemm_f32_skinny_kernel<1, kRope, TB, true, WAVES><<<dim3(blocks, 1), 64 * WAVES, 0, s>>>(x, w, (const TB*)bias, q_out, T, N, K, steps, extra);
  else
    gemm_f32_skinny_kernel<1, kRope, TB, false, WAVES><<<dim3(blocks, 1), 64 * WAVES, 0, s>>>(x, w, (const TB*)bias, q_out, T, N, K, steps, extra);
  return check_launch("sp_qkv_rope_cache_f32");
}

template <typename TB>
static int launch_qkv(hipStream_t s, const float* x, const float* w, const void* bias, float* q_out, int T, int K,
                      const SkinnyExtra& extra) {
  const int N = (extra.nq + 2 * extra.nkv) * extra.hd, blocks = (extra.nq + 2 * extra.nkv) * (extra.hd / 16);
  const int steps = (K + 15) / 16;
  // Few blocks (these rows cannot be split along K: the rotation needs whole sums): eight waves a block share K, so
  // that half as many trips to memory follow each other in a wave (14 heads of 64 at a width of 896, 72 blocks:
  // 7.8 against 8.8 us; 16 heads of 128 at 1,536, 128 blocks: 11.8 against 13.3).
  if (blocks <= 128 && steps > 32) return launch_qkv_waves<TB, 8>(s, x, w, bias, q_out, T, K, extra, N, blocks, steps);
  return launch_qkv_waves<TB, 4>(s, x, w, bias, q_out, T, K, extra, N, blocks, steps);
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

// out[T, I] (float32) = act(a . w[:I]^T) * (a . w[I:]^T), w float32 [2 I, K], up to 16 tokens: the gated product of
// a decode step on the float32 path, in one kernel.  a = x (float32 [T, K]), or rmsnorm(x) * norm_w (float32 [K],
// eps) where norm_w is given: the norm before the feed-forward folded in.
extern "C" int sp_gate_up_silu_f32(void* stream, const float* x, const float* norm_w, float eps, const float* w, float* out,
                                   int T, int I, int K, int activation) {
  SP_REQUIRE(activation == 0, "sp_gate_up_silu_f32: no kernel for activation %d (0 = SiLU)", activation);
  SP_REQUIRE(sp_gate_up_silu_f32_takes(T, I, K), "sp_gate_up_silu_f32: shape T=%d I=%d K=%d is not taken", T, I, K);
  SP_REQUIRE(x && w && out && (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(norm_w)) % 16 == 0,
             "sp_gate_up_silu_f32: operands must be given and 16-byte aligned");
  return gemm_f32_gated((hipStream_t)stream, x, norm_w, eps, w, out, T, I, K);
}

// Whether sp_qkv_rope_cache_f32 takes the shape: up to 16 tokens, head sizes in 16s turned whole, pairing "halves".
extern "C" int sp_qkv_rope_cache_f32_takes(int T, int K, int nq, int nkv, int hd, int rotary_dim, int pairing) {
  return T >= 1 && T <= 16 && K % 4 == 0 && K >= 64 && nq > 0 && nkv > 0 && hd > 0 && hd % 16 == 0 && rotary_dim == hd && pairing == 0;
}

// q, k, v = a . w^T + bias for up to 16 tokens, all float32; q and k heads turned by positions * inv_freq (angles in
// float64 where inv_freq_tail, the float64 table minus inv_freq, is given); q to q_out [T, nq * hd], k and v into the
// paged pools at slot_mapping.  a = x [T, K], or rmsnorm(x) * norm_w where norm_w is given.
extern "C" int sp_qkv_rope_cache_f32(void* stream, const float* x, const float* norm_w, float eps, const float* w,
                                     int bias_dtype, const void* bias, float* q_out, const int32_t* positions,
                                     const float* inv_freq, const float* inv_freq_tail, int rotary_dim,
                                     const int32_t* slot_mapping, float* k_pool, float* v_pool, int T, int K, int nq,
                                     int nkv, int hd, int page_size, int num_pages, int pairing) {
  SP_REQUIRE(sp_qkv_rope_cache_f32_takes(T, K, nq, nkv, hd, rotary_dim, pairing),
             "sp_qkv_rope_cache_f32: T=%d K=%d heads=%d/%d hd=%d rotary=%d pairing=%d is not taken", T, K, nq, nkv, hd,
             rotary_dim, pairing);
  SP_REQUIRE(x && w && q_out && positions && inv_freq && slot_mapping && k_pool && v_pool && page_size > 0 && num_pages > 0,
             "sp_qkv_rope_cache_f32: null operand or bad cache geometry");
  SP_REQUIRE((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(norm_w)) % 16 == 0,
             "sp_qkv_rope_cache_f32: operands must be 16-byte aligned");
  SP_REQUIRE(!bias || bias_dtype == kF32 || bias_dtype == kBF16, "sp_qkv_rope_cache_f32: unsupported bias dtype %d", bias_dtype);
  SkinnyExtra extra = {};
  extra.norm_w = norm_w; extra.eps = eps; extra.positions = positions; extra.inv_freq = inv_freq;
  extra.inv_freq_tail = inv_freq_tail; extra.slot_mapping = slot_mapping; extra.k_pool = k_pool; extra.v_pool = v_pool;
  extra.nq = nq; extra.nkv = nkv; extra.hd = hd; extra.page_size = page_size; extra.num_pages = num_pages;
  if (bias && bias_dtype == kBF16) return launch_qkv<bf16_t>((hipStream_t)stream, x, w, bias, q_out, T, K, extra);
  return launch_qkv<float>((hipStream_t)stream, x, w, bias, q_out, T, K, extra);
}
