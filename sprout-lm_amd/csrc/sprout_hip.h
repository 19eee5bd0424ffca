// C interface of libsprout_hip.so.  Every function returns 0 on success; otherwise
// sp_last_error() gives the reason.  Pointers are device pointers unless named host_*.
// dtype codes: 0 = float32, 1 = bfloat16.  All launches go to `stream`.
// Variants of an operation that parts may ask for are numbered, one `int` each; a number that no kernel
// implements is refused with an error, so another variant is an addition here and in the kernels, never a guess:
//   pairing of a rotation     0 = halves of the rotated dimensions (d with d + rotary_dim / 2, "neox")
//   activation of a gated product   0 = SiLU (x / (1 + exp(-x)))
#pragma once
#include <stdint.h>

extern "C" {

const char* sp_last_error();
int sp_version();

// residual[t, :] = table[tokens[t], :]            residual is float32 [T, H]
int sp_embed(void* stream, int table_dtype, const void* table, const int32_t* tokens, float* residual,
             int T, int H, int V);

// out[r, :] = rmsnorm(x[rows ? rows[r] : r, :]) * w      x float32 [*, H]; out [R, H] of out_dtype
int sp_rmsnorm(void* stream, const float* x, const int32_t* rows, int w_dtype, const void* w, float eps,
               int out_dtype, void* out, int R, int H);

// out = a[T, K] . w[N, K]^T (+ bias[N])
// mode 0: store as out_dtype [T, N];  mode 1: out (float32 [T, N]) += result;  mode 2: store float32
int sp_gemm(void* stream, int a_dtype, const void* a, int w_dtype, const void* w, int bias_dtype,
            const void* bias, int mode, int out_dtype, void* out, int T, int N, int K);

// Decode-sized products (T <= 64, bfloat16) with neighbouring work folded in.  Activations are x
// [T, K] bfloat16, or, with residual != null, rmsnorm(residual [T, K] float32) * norm_w computed inside.
// sp_fused_supported(kind, ...): kind 0..2 = plain modes of sp_gemm, 3 = sp_qkv_rope_cache, 4 = sp_gate_up_silu.
// `variant`: the pairing (kind 3) or the activation (kind 4) asked for; 0 otherwise.
int sp_fused_supported(int kind, int T, int N, int K, int hd, int rotary_dim, int norm, int variant);
// Whether folding the norm into the product (norm = 1 above) is faster than a norm kernel before it.
int sp_fused_norm_pays(int T, int N, int K);
// What the tiled product for many tokens would do with T x N x K, without running anything: kind 0 store,
// 1 accumulate, 2 gated (N = 2 I), 3 rotating (head size hd); plan = {block rows, block columns, splits of K,
// waves of a block}.
// Returns 1 where that kernel (for kind 3 its rotating epilogue) does not take the product.
int sp_pipe_plan(int kind, int T, int N, int K, int hd, int* plan);
// How that kernel numbers its blocks: tile_of[2 b], tile_of[2 b + 1] = token tile and weight tile of block b (which
// runs on XCD b % 8), -1 for a block with nothing to do; returns the number of blocks.  Runs nothing.
int sp_pipe_tiles(int tiles_t, int tiles_n, int* tile_of, int room);
int sp_gemm_decode(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w, float eps,
                   const void* w, int bias_dtype, const void* bias, int mode, void* out, int T, int N, int K);
// q, k, v projection (+ bias), rotation of q and k, q to q_out [T, nq * hd], k and v into the paged pools.
// With more than 64 tokens (head sizes that are multiples of 64) the tiled product does it in its epilogue;
// cos_sin (may be null): the table of sp_rope_table for these positions, which saves it the sines and cosines.
int sp_qkv_rope_cache(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w,
                      float eps, const void* w, int bias_dtype, const void* bias, void* q_out,
                      const int32_t* positions, const float* inv_freq, int rotary_dim, const int32_t* slot_mapping,
                      void* k_pool, void* v_pool, int T, int K, int nq, int nkv, int hd, int page_size,
                      const float* cos_sin, int pairing);
// out [T][half][2] = (cosine, sine) of positions[t] * inv_freq[d]: the same for every layer of a step.
int sp_rope_table(void* stream, const int32_t* positions, const float* inv_freq, int half, float* out, int T);
// out [T, I] = silu(x . w[:I]^T) * (x . w[I:]^T)
int sp_gate_up_silu(void* stream, const void* x, const float* residual, int norm_w_dtype, const void* norm_w, float eps,
                    const void* w, void* out, int T, int I, int K, int activation);

// Rotates q and k heads of qkv[T, (nq + 2 nkv) * hd] in place (neox pairing, angle = position *
// inv_freq[d]) and writes k and v of every token into the paged pools at slot_mapping[t]
// (= page * page_size + offset; negative: not written).  nkv == 0: only q is rotated.
// The key pool is [pages][nkv][page_size][hd], the value pool [pages][nkv][hd][page_size], of `dtype`.
int sp_rope_cache(void* stream, int dtype, void* qkv, const int32_t* positions, const float* inv_freq,
                  const float* inv_freq_tail, int rotary_dim, const int32_t* slot_mapping, void* k_pool, void* v_pool, int T, int nq,
                  int nkv, int hd, int page_size, int num_pages, int pairing);

// Causal attention of a mixed batch over the paged pools.
// q: [T, q_stride] (head h at column h * hd), out: [T, nq * hd].
// Sequence s owns tokens q_start[s] .. q_start[s] + q_len[s]; their positions end at ctx_len[s] - 1.
// sp_attention_plan tells how the caller must list the work: tiles [n_tiles][2] = (sequence, first
// query of the tile within the sequence's tokens) of plan[0] queries each, over every sequence
// (plan[1] == 1) or over the sequences with more than one query only, the others being listed in
// decode_seqs (plan[1] == 0; a null decode_seqs stands for sequences 0 .. n_decode - 1, each of one query, so that
// q_start[s] == s, which saves the kernels two dependent reads).  max_decode_ctx: largest ctx_len among decode_seqs; max_tile_ctx: largest
// ctx_len among the sequences of the tile list (it only guides how a long walk over the keys is shared out
// between blocks: a smaller value than the truth costs time, not correctness); mean_tile_walk: the mean over
// the tiles of the keys a tile walks (likewise a hint, 0 if unknown: where the longest walk is much longer than
// the mean, as in a prompt's first portion, a block takes a long and a short tile).
// window <= 0: all keys; else keys with position - key < window.
// workspace: sp_attention_workspace_floats(...) floats of scratch for partial results.
int sp_attention_plan(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind, int* plan);
int64_t sp_attention_workspace_floats(int dtype, int hd, int page_size, int nq, int nkv, int kernel_kind,
                                      int n_decode, int max_decode_ctx, int n_tiles, int max_tile_ctx);
// scores: what stands between q . k and the softmax, numbered like the variants above: 0 = the scaled product and
// nothing else (the one the kernels have; a cap, a bias or sinks would be further numbers, refused until written).
int sp_attention(void* stream, int dtype, const void* q, int q_stride, const void* k_pool,
                 const void* v_pool, const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                 const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles, int tile_q,
                 int max_tile_ctx, int mean_tile_walk, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                 float* workspace, int64_t workspace_floats, void* out, int nq, int nkv, int hd, int page_size,
                 int num_pages, int window, float scale, int kernel_kind, int scores);

// A step of one-query sequences only (bfloat16): attention with the output projection folded into the merge
// of the key chunks: residual[q_start[seq], :] += attention(seq) . w_o^T with w_o [hidden, nq * hd] bfloat16
// and residual float32 [rows, hidden].  sp_attention_decode_project_takes says whether a step is taken
// (several chunks of keys, at most 64 sequences, a narrow model); the workspace is sp_attention's for the step.
int sp_attention_decode_project_takes(int hd, int page_size, int nq, int nkv, int n_decode, int max_decode_ctx,
                                      int hidden);
int sp_attention_decode_project(void* stream, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                                const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                                const int32_t* ctx_len, const int32_t* decode_seqs, int n_decode, int max_decode_ctx,
                                float* workspace, int64_t workspace_floats, const void* w_o, float* residual,
                                int hidden, int nq, int nkv, int hd, int page_size, int num_pages, int window,
                                float scale, int scores);

// out[t, i] = act(gu[t, i]) * gu[t, I + i]
int sp_silu_mul(void* stream, int dtype, const void* gu, void* out, int T, int I, int activation);

// dst (dst_dtype) = src (src_dtype), n elements

// tokens[i] = previous[source[i]] for every i < n with source[i] >= 0 (others are left as they are):
// The float32 path's decode-sized products (up to 16 tokens, everything float32) with neighbouring work folded in.
// Activations are x [T, K], or rmsnorm(x) * norm_w computed inside the kernel where norm_w [K] is given.
//   sp_gate_up_silu_f32:   out[T, I] = act(a . w[:I]^T) * (a . w[I:]^T)
//   sp_qkv_rope_cache_f32: q, k, v = a . w^T + bias; q and k heads turned whole by positions * inv_freq (angles
//                          in float64 where inv_freq_tail, the float64 table minus inv_freq, is given); q to
//                          q_out [T, nq * hd], k and v into the paged pools at slot_mapping.  Head sizes in 16s.
int sp_gate_up_silu_f32_takes(int T, int I, int K);
int sp_gate_up_silu_f32(void* stream, const float* x, const float* norm_w, float eps, const float* w, float* out,
                        int T, int I, int K, int activation);
int sp_qkv_rope_cache_f32_takes(int T, int K, int nq, int nkv, int hd, int rotary_dim, int pairing);
int sp_qkv_rope_cache_f32(void* stream, const float* x, const float* norm_w, float eps, const float* w, int bias_dtype,
                          const void* bias, float* q_out, const int32_t* positions, const float* inv_freq,
                          const float* inv_freq_tail, int rotary_dim, const int32_t* slot_mapping, float* k_pool,
                          float* v_pool, int T, int K, int nq, int nkv, int hd, int page_size, int num_pages, int pairing);

// dst[i] = a seeded random value, a function of (key, first + i) alone: the sum of twelve 16-bit fields of three
// 64-bit hashes, centred, times scale (+ offset if add_offset): near normal with deviation 65536 * scale.
// weights/random_init.py computes the same numbers on the host.
int sp_random_fill(void* stream, int dtype, void* dst, int64_t n, uint64_t key, int64_t first, float scale,
                   float offset, int add_offset);

// feeds tokens sampled by a step that the host has not read yet into the next step.  previous holds at
// least max(source) + 1 entries; a value outside [0, vocab) is replaced by 0.
int sp_feed_tokens(void* stream, int32_t* tokens, const int32_t* previous, const int32_t* source, int n, int vocab);

// Greedy / temperature sampling of R rows of float32 logits [R, V].
// temperature[r] == 0: lowest index of the maximum.  Else argmax of logits / temperature + Gumbel noise
// from a counter generator keyed by (seed[r], counter[r], column).
// out[r] = token, or -1 if a logit of the row is not finite.  workspace: R * 2 * blocks_per_row floats.
int sp_sample(void* stream, const float* logits, const float* temperature, const int64_t* seed,
              const int32_t* counter, int32_t* out, float* workspace, int R, int V);
int sp_sample_workspace_floats(int R, int V);

// sp_sample for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
// harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The partial results of the first
// stage go to a device array of the library's own (sp_sample_static_max_floats() floats, 256 KiB, one copy on
// every GPU the library is used on, kept until the process ends) instead of a workspace; the call allocates and
// frees nothing.  Sizes whose partial results (sp_sample_workspace_floats(R, V)) do not fit are refused.  The
// device of `stream` must be the current device.  All calls on one GPU share that GPU's array: calls whose
// kernels may overlap (different streams, no ordering between them) race; calls on one stream do not.  What an
// earlier call left in the array is never read.
int sp_sample_static(void* stream, const float* logits, const float* temperature, const int64_t* seed,
                     const int32_t* counter, int32_t* out, int R, int V);
int sp_sample_static_max_floats();

// Probes for the benchmark's report, not used by the engine: a kernel that only reads `bytes` of `data` (16-byte
// loads from `blocks` blocks of 256 threads), and one that only multiplies on the matrix cores (`blocks` blocks of four waves,
// `iterations` x 4 independent 32x32x16 bfloat16 products a wave; *flops receives the operations of one launch).
int sp_probe_read(void* stream, const void* data, int64_t bytes, int blocks, float* sink);
int sp_probe_mfma(void* stream, int blocks, int iterations, float* sink, double* flops);
}
