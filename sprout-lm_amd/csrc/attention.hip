// Entry point of attention: checks the arguments and picks a kernel.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {
int attention_generic(hipStream_t s, int dtype, const void* q, int q_stride, const void* k_pool,
                      const void* v_pool, const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                      const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles, void* out,
                      int nq, int nkv, int hd, int page_size, int num_pages, int window, float scale, int max_tile_ctx,
                      float* workspace, bool single);
size_t attention_generic_workspace_floats(int dtype, int page_size, int n_tiles, int nq, int nkv, int hd, int max_tile_ctx,
                                          bool single);
int attention_generic_tile_q(int dtype, int nq, int nkv, int hd, int page_size);
bool attention_mfma_supports(int hd, int page_size, int nq, int nkv);
bool attention_mfma_decode_supports(int nq, int nkv);
int attention_mfma_tile_q(int hd);
size_t attention_decode_workspace_floats(int n_decode, int nq, int hd, int max_ctx);
size_t attention_prefill_workspace_floats(int n_tiles, int nq, int nkv, int hd, int page_size, int max_tile_ctx);
int attention_mfma(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                   const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* q_len,
                   const int32_t* ctx_len, const int32_t* tiles, int n_tiles, const int32_t* decode_seqs, int n_decode,
                   int max_decode_ctx, int max_tile_ctx, int mean_tile_walk, float* workspace, void* out, int nq, int nkv,
                   int hd, int page_size, int num_pages, int window, float scale);
bool attention_decode_project_takes(int hd, int page_size, int nq, int nkv, int n_decode, int max_decode_ctx, int hidden);
int attention_mfma_decode_project(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                  const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                                  const int32_t* ctx_len, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                                  float* workspace, const void* w_o, float* residual, int hidden, int nq, int nkv,
                                  int hd, int page_size, int num_pages, int window, float scale);
}  // namespace sprout

using namespace sprout;

// kernel_kind: 0 = the engine's choice, 1 = the float32-arithmetic kernel.
static bool use_mfma(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind) {
  return kernel_kind == 0 && dtype == kBF16 && nkv > 0 && nq % nkv == 0 && attention_mfma_supports(hd, page_size, nq, nkv);
}

// What the chosen kernel wants of the caller.
//   plan[0]: queries per tile of the tile list
//   plan[1]: 1 if the tile list holds every sequence, 0 if only sequences with more than one query
//            (the others are then given as `decode_seqs`)
extern "C" int sp_attention_plan(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind, int* plan) {
  if (use_mfma(dtype, hd, page_size, nq, nkv, kernel_kind)) {
    plan[0] = attention_mfma_tile_q(hd);
    plan[1] = attention_mfma_decode_supports(nq, nkv) ? 0 : 1;
  } else {
    plan[0] = attention_generic_tile_q(dtype, nq, nkv, hd, page_size);
    plan[1] = 1;
  }
  return 0;
}

static int64_t workspace_floats_of(int hd, int page_size, int nq, int nkv, int n_decode, int max_decode_ctx,
                                   int n_tiles, int max_tile_ctx) {
  const size_t decode = attention_mfma_decode_supports(nq, nkv)
                            ? attention_decode_workspace_floats(n_decode, nq, hd, max_decode_ctx) : 0;
  return (int64_t)(decode + attention_prefill_workspace_floats(n_tiles, nq, nkv, hd, page_size, max_tile_ctx));
}

extern "C" int64_t sp_attention_workspace_floats(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind,
                                                 int n_decode, int max_decode_ctx, int n_tiles, int max_tile_ctx) {
  if (!use_mfma(dtype, hd, page_size, nq, nkv, kernel_kind))   // (n_decode == n_tiles: every sequence brings one query)
    return (int64_t)attention_generic_workspace_floats(dtype, page_size, n_tiles, nq, nkv, hd, max_tile_ctx, n_decode > 0 && n_decode == n_tiles);
  return workspace_floats_of(hd, page_size, nq, nkv, n_decode, max_decode_ctx, n_tiles, max_tile_ctx);
}

extern "C" int sp_attention(void* stream, int dtype, const void* q, int q_stride, const void* k_pool,
                            const void* v_pool, const int32_t* block_tables, int max_blocks,
                            const int32_t* q_start, const int32_t* q_len, const int32_t* ctx_len,
                            const int32_t* tiles, int n_tiles, int tile_q, int max_tile_ctx, int mean_tile_walk,
                            const int32_t* decode_seqs, int n_decode, int max_decode_ctx, float* workspace,
                            int64_t workspace_floats, void* out, int nq,
                            int nkv, int hd, int page_size, int num_pages, int window, float scale, int kernel_kind,
                            int scores) {
  SP_REQUIRE(scores == 0, "sp_attention: no kernel for score stage %d (0 = the scaled product alone)", scores);
  SP_REQUIRE(dtype == kF32 || dtype == kBF16, "sp_attention: unsupported dtype %d", dtype);
  SP_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "sp_attention: %d query heads do not divide into %d groups", nq, nkv);
  SP_REQUIRE(hd > 0 && hd <= 512, "sp_attention: head size %d is outside 1..512", hd);
  SP_REQUIRE(page_size > 0 && num_pages > 0 && max_blocks > 0, "sp_attention: bad cache geometry");
  SP_REQUIRE(q_stride >= nq * hd, "sp_attention: q row stride %d is smaller than %d", q_stride, nq * hd);
  int plan[2];
  sp_attention_plan(dtype, hd, page_size, nq, nkv, kernel_kind, plan);
  SP_REQUIRE(tile_q == plan[0], "sp_attention: tiles were built for %d queries, the kernel takes %d", tile_q, plan[0]);
  // a kernel that takes every sequence in its tile list may be told that each brings one query: n_decode == n_tiles
  SP_REQUIRE(plan[1] == 0 || n_decode == 0 || (n_decode == n_tiles && !decode_seqs),
             "sp_attention: this kernel takes every sequence in the tile list");
  SP_REQUIRE(n_tiles >= 0 && n_decode >= 0 && (n_tiles == 0 || tiles), "sp_attention: missing tile list");
  hipStream_t s = (hipStream_t)stream;
  if (!use_mfma(dtype, hd, page_size, nq, nkv, kernel_kind)) {
    if (n_tiles == 0) return 0;
    SP_REQUIRE(max_tile_ctx >= 0, "sp_attention: negative context length");
    const bool single = n_decode > 0 && n_decode == n_tiles;
    const int64_t need = (int64_t)attention_generic_workspace_floats(dtype, page_size, n_tiles, nq, nkv, hd, max_tile_ctx, single);
    SP_REQUIRE(need == 0 || (workspace && workspace_floats >= need),
               "sp_attention: workspace of %lld floats is smaller than the %lld needed", (long long)workspace_floats,
               (long long)need);
    return attention_generic(s, dtype, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, q_len,
                             ctx_len, tiles, n_tiles, out, nq, nkv, hd, page_size, num_pages, window, scale,
                             max_tile_ctx, need ? workspace : nullptr, single);
  }
  SP_REQUIRE(max_decode_ctx >= 0 && max_decode_ctx <= max_blocks * page_size,
             "sp_attention: decode context %d exceeds the block tables", max_decode_ctx);
  SP_REQUIRE(max_tile_ctx >= 0, "sp_attention: negative context length");
  const int64_t need = workspace_floats_of(hd, page_size, nq, nkv, n_decode, max_decode_ctx, n_tiles, max_tile_ctx);
  SP_REQUIRE(need == 0 || (workspace && workspace_floats >= need),
             "sp_attention: workspace of %lld floats is smaller than the %lld needed", (long long)workspace_floats,
             (long long)need);
  return attention_mfma(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, q_len, ctx_len, tiles,
                        n_tiles, decode_seqs, n_decode, max_decode_ctx, max_tile_ctx,
                        mean_tile_walk > 0 ? mean_tile_walk : max_tile_ctx, workspace, out,
                        nq, nkv, hd, page_size, num_pages, window, scale);
}

// Whether sp_attention_decode_project takes a step of n_decode one-query sequences (bfloat16 only).
extern "C" int sp_attention_decode_project_takes(int hd, int page_size, int nq, int nkv, int n_decode,
                                                 int max_decode_ctx, int hidden) {
  return nq > 0 && nkv > 0 && nq % nkv == 0 &&
         attention_decode_project_takes(hd, page_size, nq, nkv, n_decode, max_decode_ctx, hidden);
}

// A step of one-query sequences only, bfloat16: attention and the output projection w_o [hidden, nq * hd]
// (bfloat16, no bias) in one: residual[q_start[seq], :] += attention(seq) . w_o^T, residual float32
// [rows, hidden].  The workspace is the one of sp_attention for the same step.
extern "C" int sp_attention_decode_project(void* stream, const void* q, int q_stride, const void* k_pool,
                                           const void* v_pool, const int32_t* block_tables, int max_blocks,
                                           const int32_t* q_start, const int32_t* ctx_len, const int32_t* decode_seqs,
                                           int n_decode, int max_decode_ctx, float* workspace, int64_t workspace_floats,
                                           const void* w_o, float* residual, int hidden, int nq, int nkv, int hd,
                                           int page_size, int num_pages, int window, float scale, int scores) {
  SP_REQUIRE(scores == 0, "sp_attention_decode_project: no kernel for score stage %d (0 = the scaled product alone)", scores);
  SP_REQUIRE(sp_attention_decode_project_takes(hd, page_size, nq, nkv, n_decode, max_decode_ctx, hidden),
             "sp_attention_decode_project: hd=%d page=%d heads=%d/%d sequences=%d context=%d hidden=%d is not taken",
             hd, page_size, nq, nkv, n_decode, max_decode_ctx, hidden);
  SP_REQUIRE(q && k_pool && v_pool && block_tables && q_start && ctx_len && w_o && residual,
             "sp_attention_decode_project: null operand");
  SP_REQUIRE(page_size > 0 && num_pages > 0 && max_blocks > 0 && max_decode_ctx <= max_blocks * page_size,
             "sp_attention_decode_project: decode context %d exceeds the block tables", max_decode_ctx);
  SP_REQUIRE(q_stride >= nq * hd, "sp_attention_decode_project: q row stride %d is smaller than %d", q_stride, nq * hd);
  const int64_t need = workspace_floats_of(hd, page_size, nq, nkv, n_decode, max_decode_ctx, 0, 0);
  SP_REQUIRE(workspace && workspace_floats >= need,
             "sp_attention_decode_project: workspace of %lld floats is smaller than the %lld needed",
             (long long)workspace_floats, (long long)need);
  return attention_mfma_decode_project((hipStream_t)stream, q, q_stride, k_pool, v_pool, block_tables, max_blocks,
                                       q_start, ctx_len, decode_seqs, n_decode, max_decode_ctx, workspace, w_o, residual,
                                       hidden, nq, nkv, hd, page_size, num_pages, window, scale);
}
