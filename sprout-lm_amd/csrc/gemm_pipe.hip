// The plain modes of the pipelined tiled product (store, accumulate, store float32), its shapes and the choice
// between them.  The kernel itself is in gemm_pipe.h; the products with a bfloat16 bias are instantiated in
// gemm_pipe_bias16.hip, the gated and the rotating epilogue in gemm_pipe_epilogues.hip, so that the parts compile
// side by side.
#include "gemm_pipe.h"

namespace sprout {

// Whether the pipelined kernel takes the shape: whole steps of 64 along K, and tile offsets that fit 32 bits.
bool gemm_pipe_takes(int T, int N, int K) {
  return K % 64 == 0 && K >= 64 && size_t(256) * K * 2 < (size_t(1) << 31) && size_t(N) * K * 2 < (size_t(1) << 32);
}

// Tile shapes of the pipelined kernel, largest first, with what was measured of them on a full chip:
// microseconds per step of 64 along K and block, blocks per CU (LDS), and bytes a block fetches per step.
struct PipeShape { int bm, bn, per_cu; float short_us, long_us; };   // a step of a walk of up to 16 steps, of a longer one
static const PipeShape kPipeShapes[] = {
    {256, 256, 1, 2.05f, 2.05f},   // 8 waves, 2 stages
    {256, 128, 1, 1.4f, 1.05f},    // 8 waves, 3 stages (on 4 waves of 128 x 64 sums each: 1.25 us)
    {128, 128, 1, 0.72f, 0.64f},   // 8 waves, 4 stages (on 4 waves: 0.72 us)
    {64, 64, 2, 0.41f, 0.5f},      // 4 waves, 4 stages
    {64, 256, 1, 0.75f, 0.75f},    // 8 waves, 3 stages (few tokens)
    // two blocks of 64 x 128 on a CU get in each other's way on a long K (measured at 56 and 296 steps)
    {64, 128, 2, 0.7f, 0.8f},      // 4 waves, 3 stages (few tokens)
    {384, 256, 1, 3.3f, 3.3f},     // 8 waves, 2 stages (all of the LDS): where it saves a round of blocks
    {64, 64, 2, 0.45f, 0.45f},     // 2 waves with two tile columns each, 4 stages (few tokens: most blocks)
    // 4 waves in a column, five tile columns each, 3 stages: where 256 x 256 leaves CUs idle; with a short K its
    // blocks cost more than their share (9,728 rows, K = 896: 57 us against 51)
    {256, 160, 1, 2.0f, 1.4f},
};

// Picks the shape and the split of K with the least estimated time.  Fetching tiles from L2 bounds these
// kernels, so large tiles win whenever they still fill the chip; products with few tiles (narrow outputs)
// take small tiles or, when accumulating, a split of K, whose float atomics are charged per element.
void pipe_choice(int T, int N, int K, bool may_split, int* shape, int* splits, bool paired) {
  const int steps = K / 64;
  float best = 1e30f;
  *shape = 2;
  *splits = 1;
  if (T <= 64) {
    // Few tokens: the weights are read once from memory, which bounds the product from below; a block's
    // steps follow each other at memory latency, so K is split until the blocks are short enough.
    const float stream_us = float(N) * float(K) * 2.f / 4.5e6f;
    for (int c : {4, 5, 7}) {
      const PipeShape& p = kPipeShapes[c];
      const int tiles = (N + p.bn - 1) / p.bn, slots = 256 * p.per_cu;
      for (int sp : {1, 2, 4, 8, 16}) {
        if (sp > 1 && (!may_split || steps / sp < 8)) break;
        // blocks of two waves do badly on a long walk along K (37,888 x 3,584 at 64 tokens: 66 us against 59)
        if (c == 7 && steps / sp > 24) continue;
        const int rounds = (tiles * sp + slots - 1) / slots;
        // a CU pulls about 30 GB/s of weight rows, however many blocks it holds: the CU with the most blocks
        const float pull_us = float((tiles * sp + 255) / 256) * float(p.bn) * float(K / sp) * 2.f / 30e3f;
        float t = fmaxf(fmaxf(stream_us, pull_us), rounds * float((steps + sp - 1) / sp) * p.short_us) + 2.0f;
        if (sp > 1) t += 2.7e-6f * float(T) * float(N) * sp;
        if (t < best) { best = t; *shape = c; *splits = sp; }
      }
    }
    return;
  }
  for (int c : {0, 1, 2, 3, 5, 6, 8}) {
    // (64 x 128 fills the chip where 128 x 128 leaves CUs idle and 64 x 64 needs a second round: 2,048 tokens,
    // 1,152 rows, K = 896: 14.8 us against 17.2 and 15.1)
    if (c == 3 && paired) continue;   // one tile column a wave: no lane holds both of a pair
    // 256 x 160: an odd number of tile columns a wave pairs nothing either.  (2,048 tokens, K = 3,584: 4,608 rows
    // make 232 blocks instead of 144 of 256 x 256, 83 us against 91; 5,120 rows at K = 27,648 make 256 instead of 160,
    // 607 us against 658; with a short K its blocks cost more than their share, 57 us against 51 at 9,728 rows, K = 896)
    if (c == 8 && paired) continue;
    const PipeShape& p = kPipeShapes[c];
    // blocks of 384 x 256, with all of the LDS in two stages, fetch slowly on a long K once there are more
    // token tiles than the 8 that run together on an XCD (4,096 tokens, 4,608 rows, K = 3,584: 241 us against 180
    // on 256 x 256, for all the round of blocks they save; with one token tile, 264 tokens, 55,296 rows,
    // K = 5,120, their 253 us are the best there is)
    // (64 x 128 on a short K beside many tokens: 256 tokens, 9,728 rows, K = 896 with the gating: 16.3 us against
    // 13.8 on 128 x 128)
    const float step_us = steps <= 16 ? (c == 5 ? 0.8f : p.short_us) : (c == 6 && (T + p.bm - 1) / p.bm > 8) ? 4.3f : p.long_us;
    // Blocks are counted on the XCD that holds the most, as the kernel numbers them: XCD c runs the weight tiles
    // c, c + 8, ... with all their token tiles and splits on its 32 CUs, and an equal run of the blocks of the
    // weight tiles that are left over (264 tokens, 3,584 rows, K = 18,944 on 128 x 128 with K in three: 252
    // blocks in all, which were 36 on XCD 0 before the left-over tiles were dealt out: a second round, 106 us
    // where 256 x 128 with K in four, 32 a XCD, takes 89).
    const PipeTiles tiles = pipe_tiles((T + p.bm - 1) / p.bm, (N + p.bn - 1) / p.bn);
    const int slots = 32 * p.per_cu;
    for (int sp : {1, 2, 3, 4, 6, 8}) {
      if (sp > 1 && (!may_split || steps / sp < 8)) break;
      const int blocks = (tiles.full * tiles.tiles_t + tiles.run) * sp, full = blocks / slots, rest = blocks % slots;
      const float per_block = float((steps + sp - 1) / sp) * step_us + 1.0f;
      // a round that does not fill the chip runs somewhat faster: fewer blocks share the caches; much faster for
      // the blocks of 384 x 256 with one tile of tokens, whose two stages hold all of the LDS and wait for their tiles
      // the most (264 tokens, 37,888 rows, K = 3,584 with the gating: 148 blocks take 2.25 us a step, 126 us
      // against 134 on 128 x 128)
      const float alone = c == 6 && full == 0 && T <= p.bm ? 0.3f : 0.7f;
      float t = full * per_block + (rest ? per_block * (alone + (1.f - alone) * float(rest) / slots) : 0.f);
      if (sp > 1) t += 2.7e-6f * float(T) * float(N) * sp;      // float atomics into the output
      if (t < best) { best = t; *shape = c; *splits = sp; }
    }
  }
}

int gemm_bf16_pipe_bias16(hipStream_t s, const void* a, const void* w, const void* bias, int mode, void* out, int T, int N, int K);

int gemm_bf16_pipe(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                   int T, int N, int K) {
  if (bias && bias_dtype == kBF16) return gemm_bf16_pipe_bias16(s, a, w, bias, mode, out, T, N, K);
  return pipe_shape<float>(s, a, w, bias, mode, out, T, N, K);
}

}  // namespace sprout
