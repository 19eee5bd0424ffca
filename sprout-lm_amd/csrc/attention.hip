// Entry point of attention: checks the arguments and picks a kernel.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {
int attention_generic(hipStream_t s, int dtype, const void* q, int q_stride, const void* k_pool,
                      const void* v_pool, const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                      const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles, void* out,
                      int nq, int nkv, int hd, int page_size, int num_pages, int window, float scale);
}  // namespace sprout

using namespace sprout;

// kernel_kind: 0 = the engine's choice, 1 = the float32-arithmetic kernel.
extern "C" int sp_attention_tile_q(int dtype, int hd, int max_q_len, int kernel_kind) { return 16; }

extern "C" int sp_attention(void* stream, int dtype, const void* q, int q_stride, const void* k_pool,
                            const void* v_pool, const int32_t* block_tables, int max_blocks,
                            const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                            const int32_t* tiles, int n_tiles, int tile_q, void* out, int nq, int nkv, int hd,
                            int page_size, int num_pages, int window, float scale, int kernel_kind) {
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_attention: unsupported dtype %d", dtype);
  SP_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "sp_attention: %d query heads do not divide into %d groups", nq, nkv);
  SP_REQUIRE(hd > 0 && hd <= 256, "sp_attention: head size %d is outside 1..256", hd);
  SP_REQUIRE(page_size > 0 && num_pages > 0 && max_blocks > 0, "sp_attention: bad cache geometry");
  SP_REQUIRE(q_stride >= nq * hd, "sp_attention: q row stride %d is smaller than %d", q_stride, nq * hd);
  SP_REQUIRE(tile_q == sp_attention_tile_q(dtype, hd, 0, kernel_kind), "sp_attention: tiles were built for %d queries", tile_q);
  if (n_tiles == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  return attention_generic(s, dtype, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, q_len,
                           ctx_len, tiles, n_tiles, out, nq, nkv, hd, page_size, num_pages, window, scale);
}
