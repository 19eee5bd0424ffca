// The pipelined tiled product with the gated (gate/up + SiLU) and the rotating (q/k/v + rotation + cache write)
// epilogue: the kernel of gemm_pipe.h in the shapes that gemm_pipe.hip's cost model picks.
#include "gemm_pipe.h"

namespace sprout {

// out[T, I] = silu(x . w[:I]^T) * (x . w[I:]^T): a block's weight rows are half gate rows, half the matching up rows.
int gemm_bf16_pipe_silu(hipStream_t s, const void* x, const void* w, void* out, int T, int I, int K) {
  const uint16_t *xp = (const uint16_t*)x, *wp = (const uint16_t*)w;
  int shape, splits;
  pipe_choice(T, 2 * I, K, false, &shape, &splits, true);
  if (shape == 0) return launch_pipe_mode<4, 2, 2, 4, 2, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
  if (shape == 1) return launch_pipe_mode<2, 2, 4, 2, 3, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
  if (shape == 4) return launch_pipe_mode<1, 2, 2, 4, 3, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
  if (shape == 5) return launch_pipe_mode<1, 2, 2, 2, 3, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
  if (shape == 6) return launch_pipe_mode<6, 2, 2, 4, 2, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
  if (shape == 7) return launch_pipe_mode<1, 2, 2, 1, 4, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
  return launch_pipe_mode<1, 2, 4, 2, 4, kSilu, float>(s, 1, xp, wp, nullptr, out, T, I, K, K);
}

// The block shape on which the rotating epilogue runs, or -1 where the plain product and a rotation kernel after
// it do better.  It follows the plain product's choice where that pairs tile columns (256 x 128, 128 x 128,
// 64 x 128).  Blocks of 64 x 64 have one tile column a wave and pair nothing: there 64 x 128 takes the rotation
// once its blocks fill half of the chip (14 + 2 + 2 heads of 64 at K = 896, 1,024
// tokens: 14.5 us against 17.6 apart, 512 tokens: 15.2 against 13.8; 28 + 4 + 4 heads of 128 at K = 3,584, 256
// tokens: 36.5 against 42.5).  The blocks of 256 x 256 hold 128 sums per lane, all the registers a lane has there:
// the epilogue's own would be spilled (measured at 28 + 4 + 4 heads of 128, 2,048 tokens: 332 us against 106 and a
// rotation kernel of 18), and 256 x 160 has five tile columns a wave.
static int rope_shape(int T, int N, int K) {
  int shape, splits;
  pipe_choice(T, N, K, false, &shape, &splits);
  if (shape == 3 && ((T + 63) / 64) * ((N + 127) / 128) >= 128) shape = 5;
  // (and with the rotation 128 x 128 on 8 waves beats 64 x 128 on 4 once its blocks fill half of the chip: 14 + 2 + 2
  // heads of 64 at K = 896, 2,048 tokens: 20.2 us against 23.0; 1,024 tokens: 19.2 against 14.5)
  if (shape == 5 && ((T + 127) / 128) * ((N + 127) / 128) >= 128) shape = 2;
  return shape == 1 || shape == 2 || shape == 5 ? shape : -1;
}

// q, k, v = x . w^T + bias with w [(nq + 2 nkv) * hd, K]; q and k heads rotated; q to q_out [T, nq * hd], k and v
// into the paged pools.  Head sizes that are multiples of 64, more than 64 tokens.
template <typename TB>
static int pipe_rope(hipStream_t s, const uint16_t* x, const uint16_t* w, const TB* bias, void* q_out, int T, int N, int K,
                     const RopeArgs& rope) {
  const int shape = rope_shape(T, N, K);
  if (shape == 1) return launch_pipe_mode<2, 2, 4, 2, 3, kRope, TB>(s, 1, x, w, bias, q_out, T, N, K, K, rope);
  if (shape == 2) return launch_pipe_mode<1, 2, 4, 2, 4, kRope, TB>(s, 1, x, w, bias, q_out, T, N, K, K, rope);
  if (shape == 5) return launch_pipe_mode<1, 2, 2, 2, 3, kRope, TB>(s, 1, x, w, bias, q_out, T, N, K, K, rope);
  set_error("sp_qkv_rope_cache: no rotating epilogue for %d tokens, %d rows, K = %d", T, N, K);
  return 1;
}

bool gemm_pipe_rope_takes(int T, int N, int K, int hd) {
  return T > 64 && hd % 64 == 0 && N % hd == 0 && gemm_pipe_takes(T, N, K) && rope_shape(T, N, K) >= 0;
}

// Rows and columns of every block shape, by its index in gemm_pipe.hip's list.
static const int kShapeRows[] = {256, 256, 128, 64, 64, 64, 384, 64, 256};
static const int kShapeCols[] = {256, 128, 128, 64, 256, 128, 256, 64, 160};
static const int kShapeWaves[] = {8, 8, 8, 4, 8, 4, 8, 2, 4};

}  // namespace sprout

// What the pipelined product would do with T x N x K: kind 0 store, 1 accumulate, 2 gated (N = 2 I rows of w),
// 3 rotating (head size hd).  plan = {block rows, block columns, splits of K, waves of a block}.  Returns 1 where the pipelined kernel
// (for kind 3: its rotating epilogue) does not take the product, else 0.  Runs nothing: for tests and tools.
extern "C" int sp_pipe_plan(int kind, int T, int N, int K, int hd, int* plan) {
  using namespace sprout;
  if (T < 1 || N < 1 || K < 1 || kind < 0 || kind > 3 || !plan || !gemm_pipe_takes(T, N, K)) return 1;
  int shape, splits = 1;
  if (kind == 3) {
    if (!gemm_pipe_rope_takes(T, N, K, hd)) return 1;
    shape = rope_shape(T, N, K);
  } else {
    pipe_choice(T, N, K, kind == 1, &shape, &splits, kind == 2);
  }
  if (shape < 0 || shape >= int(sizeof(kShapeRows) / sizeof(kShapeRows[0]))) return 1;
  plan[0] = kShapeRows[shape];
  plan[1] = kShapeCols[shape];
  plan[2] = splits;
  plan[3] = kShapeWaves[shape];
  return 0;
}

// The tile of every block of a launch over tiles_t token tiles and tiles_n weight tiles, as the kernel numbers them:
// tile_of[2 b] = token tile and tile_of[2 b + 1] = weight tile of block b, both -1 for a block with nothing to do.
// Returns the number of blocks (8 for each place on an XCD), or -1; writes at most `room` blocks.  Runs nothing.
extern "C" int sp_pipe_tiles(int tiles_t, int tiles_n, int* tile_of, int room) {
  using namespace sprout;
  if (tiles_t < 1 || tiles_n < 1 || !tile_of) return -1;
  const PipeTiles tiles = pipe_tiles(tiles_t, tiles_n);
  const int blocks = 8 * (tiles.own + tiles.run);
  for (int b = 0; b < blocks && b < room; ++b)
    if (!pipe_tile_of(tiles, b, &tile_of[2 * b], &tile_of[2 * b + 1])) tile_of[2 * b] = tile_of[2 * b + 1] = -1;
  return blocks;
}

namespace sprout {

int gemm_bf16_pipe_rope(hipStream_t s, const void* x, const void* w, int bias_dtype, const void* bias, void* q_out,
                        const int32_t* positions, const float* inv_freq, const int32_t* slot_mapping, void* k_pool,
                        void* v_pool, int T, int K, int nq, int nkv, int hd, int page_size, const float* table) {
  RopeArgs rope = {positions, inv_freq, slot_mapping, (uint16_t*)k_pool, (uint16_t*)v_pool, nq, nkv, hd, page_size,
                   reinterpret_cast<const float2*>(table)};
  const int N = (nq + 2 * nkv) * hd;
  if (bias && bias_dtype == kBF16)
    return pipe_rope<bf16_t>(s, (const uint16_t*)x, (const uint16_t*)w, (const bf16_t*)bias, q_out, T, N, K, rope);
  return pipe_rope<float>(s, (const uint16_t*)x, (const uint16_t*)w, (const float*)bias, q_out, T, N, K, rope);
}

}  // namespace sprout
