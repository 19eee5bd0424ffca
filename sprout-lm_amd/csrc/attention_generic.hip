// Causal grouped-query attention of a mixed batch over paged keys and values, float32 arithmetic.
// Any head size up to 512, any page size, any number of heads and groups, optional window.
// One block works on 16 queries of one sequence and one head, walking the keys 32 at a time with a
// running maximum and sum (all float32).  Keys are always walked from a multiple of 32, so the order
// of the sums at a position does not depend on how the tokens were cut into steps.
// GROUPED (a step in which every sequence brings one query): the 16 rows of a block are the query heads of one
// key/value head instead (groups of up to 16), so a group's keys and values are fetched once, not once per head.
// A step of few tiles and long contexts (decoding) would leave most of the chip idle: the keys are then
// shared out in chunks (a multiple of 32 keys each) over gridDim.z blocks, which leave their maxima, sums
// and unnormalised outputs in a workspace, and a second kernel joins them in the order of the chunks.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

constexpr int AQ = 16;  // queries per block
constexpr int AK = 32;  // keys per iteration

// One 32-key tile of keys or values of a sequence, from the pages into registers (element i of the tile is
// thread i % 256's i / 256-th).  All loads of a thread are requested before any is used.  Keys lie
// [slot][head size] inside a page, values [head size][slot]: neighbouring threads take neighbouring addresses.
// Quotient and remainder by a divisor known only at run time, for 0 <= x < 2^24, without the long
// instruction sequence of an integer division: a float product, then one step of correction either way.
struct Divider {
  int d;
  float inv;
  __device__ __forceinline__ void set(int divisor) { d = divisor; inv = 1.0f / float(divisor); }
  __device__ __forceinline__ void divmod(int x, int& q, int& r) const {
    q = int(float(x) * inv);
    r = x - q * d;
    if (r < 0) { r += d; --q; }
    if (r >= d) { r -= d; ++q; }
  }
};

struct TileSource {
  const int32_t* bt;
  int nkv, g, hd, page_size, num_pages, max_blocks, k_lo, k_end;
  Divider by_hd, by_page;
};

template <typename T, int MAXD, bool VALUES>
__device__ __forceinline__ void load_tile(const TileSource& src, const T* __restrict__ pool, int kb, float (&tmp)[2 * MAXD]) {
#pragma unroll
  for (int u = 0; u < 2 * MAXD; ++u) {
    const int i = threadIdx.x + 256 * u;
    float v = 0.f;
    if (i < AK * src.hd) {
      int jj = i % AK, d = i / AK;
      if (!VALUES) src.by_hd.divmod(i, jj, d);
      const int j = kb + jj;
      if (j >= src.k_lo && j < src.k_end) {
        int logical, slot;
        src.by_page.divmod(j, logical, slot);
        const int page = logical < src.max_blocks ? src.bt[logical] : -1;   // never past the sequence's table row
        if (page >= 0 && page < src.num_pages) {
          const size_t base = (size_t(page) * src.nkv + src.g) * src.page_size * src.hd;
          v = to_float(pool[base + (VALUES ? size_t(d) * src.page_size + slot : size_t(slot) * src.hd + d)]);
        }
      }
    }
    tmp[u] = v;
  }
}

template <int MAXD, bool VALUES>
__device__ __forceinline__ void store_tile(float* KVs, int hd, const Divider& by_hd, const float (&tmp)[2 * MAXD]) {
#pragma unroll
  for (int u = 0; u < 2 * MAXD; ++u) {
    const int i = threadIdx.x + 256 * u;
    if (i < AK * hd) {
      int jj = i % AK, d = i / AK;
      if (!VALUES) by_hd.divmod(i, jj, d);
      KVs[jj * (hd + 1) + d] = tmp[u];
    }
  }
}

template <typename T, int MAXD, bool GROUPED>  // MAXD = ceil(hd / 16) upper bound
__global__ __launch_bounds__(256) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ tiles,
    T* __restrict__ out, int nq, int nkv, int hd, int page_size, int num_pages, int window, float scale,
    float* __restrict__ part, int chunk) {
  extern __shared__ float lds[];
  // rows one float longer than their content: the four query rows that a wave reads at the same column
  // then lie in different LDS banks
  float* Qs = lds;                         // [AQ][hd + 1]
  float* KVs = Qs + AQ * (hd + 1);         // [AK][hd + 1]
  float* Ps = KVs + AK * (hd + 1);         // [AQ][AK + 1]
  const int kv_stride = hd + 1;
  constexpr int PS = AK + 1;

  const int seq = tiles[2 * blockIdx.x], q_off = tiles[2 * blockIdx.x + 1];
  const int G = nq / nkv;
  const int qlen = q_len[seq], ctx = ctx_len[seq], qs = q_start[seq];
  // rows: GROUPED the heads blockIdx.y * G .. + G - 1 of the tile's one query; else the tile's queries of head blockIdx.y
  const int nvalid = GROUPED ? (qlen - q_off > 0 ? G : 0) : min(AQ, qlen - q_off);
  if (nvalid <= 0) return;
  const int pos0 = ctx - qlen + q_off;

  for (int i = threadIdx.x; i < AQ * hd; i += 256) {
    const int r = i / hd, d = i % hd;
    const size_t at = GROUPED ? size_t(qs + q_off) * q_stride + (blockIdx.y * G + r) * hd + d
                              : size_t(qs + q_off + r) * q_stride + blockIdx.y * hd + d;
    Qs[r * kv_stride + d] = r < nvalid ? to_float(q[at]) : 0.f;
  }

  const int r = threadIdx.x / 16, c16 = threadIdx.x % 16;
  const int h = GROUPED ? blockIdx.y * G + min(r, G - 1) : blockIdx.y;      // this thread's row's head
  const int my_pos = GROUPED ? pos0 : pos0 + r;
  TileSource src;
  src.bt = block_tables + size_t(seq) * max_blocks;
  src.nkv = nkv; src.g = GROUPED ? blockIdx.y : blockIdx.y / G; src.hd = hd; src.page_size = page_size; src.num_pages = num_pages; src.max_blocks = max_blocks;
  // one past the last visible key of the tile (GROUPED: its rows are heads of one query, at pos0)
  src.k_end = pos0 + (GROUPED ? 1 : nvalid);
  src.k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int n_chunks = gridDim.z, first_key = blockIdx.z * chunk;   // this block's keys: first_key .. + chunk - 1
  if (blockIdx.z + 1 < n_chunks) src.k_end = min(src.k_end, first_key + chunk);   // the last chunk: all that is left
  src.by_hd.set(hd);
  src.by_page.set(page_size);
  const int k_lo = src.k_lo, k_end = src.k_end;
  float m = -INFINITY, l = 0.f;
  float acc[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) acc[i] = 0.f;

  // The keys and values of a tile are requested while the tile before it is still being summed: the walk
  // waits for memory once per tile, not once per element.
  float ktile[2 * MAXD], vtile[2 * MAXD];
  const int kb0 = max((k_lo / AK) * AK, first_key);
  if (kb0 < k_end) {
    load_tile<T, MAXD, false>(src, k_pool, kb0, ktile);
    load_tile<T, MAXD, true>(src, v_pool, kb0, vtile);
  }
  for (int kb = kb0; kb < k_end; kb += AK) {
    __syncthreads();  // Qs written / previous V tile consumed
    store_tile<MAXD, false>(KVs, hd, src.by_hd, ktile);
    __syncthreads();
    float s[2];
    float row_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = c16 + 16 * u, j = kb + c;
      float dot = 0.f;
#pragma unroll 8   // several LDS reads on their way at a time; the order of the sum stays
      for (int d = 0; d < hd; ++d) dot = fmaf(Qs[r * kv_stride + d], KVs[c * kv_stride + d], dot);
      const bool visible = r < nvalid && j >= k_lo && j <= my_pos && (window <= 0 || my_pos - j < window);
      s[u] = visible ? dot * scale : -INFINITY;
      row_max = fmaxf(row_max, s[u]);
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) row_max = fmaxf(row_max, __shfl_xor(row_max, o, 64));
    const float m_new = fmaxf(m, row_max);
    float alpha = 1.f, row_sum = 0.f;
    float p[2] = {0.f, 0.f};
    if (m_new != -INFINITY) {
      alpha = m == -INFINITY ? 0.f : expf(m - m_new);
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        p[u] = s[u] == -INFINITY ? 0.f : expf(s[u] - m_new);
        row_sum += p[u];
      }
    }
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) row_sum += __shfl_xor(row_sum, o, 64);
    l = l * alpha + row_sum;
    m = m_new;
    Ps[r * PS + c16] = p[0];
    Ps[r * PS + c16 + 16] = p[1];
    __syncthreads();  // scores done with the K tile; Ps complete
    store_tile<MAXD, true>(KVs, hd, src.by_hd, vtile);
    if (kb + AK < k_end) {
      load_tile<T, MAXD, false>(src, k_pool, kb + AK, ktile);
      load_tile<T, MAXD, true>(src, v_pool, kb + AK, vtile);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MAXD; ++i) {
      const int d = c16 + 16 * i;
      if (d < hd) {
        float sum = acc[i] * alpha;
#pragma unroll
        for (int c = 0; c < AK; ++c) sum = fmaf(Ps[r * PS + c], KVs[c * kv_stride + d], sum);
        acc[i] = sum;
      }
    }
  }
  if (n_chunks > 1) {
    // [tile][row][head][chunk][hd + 2]: the unnormalised output, the maximum and the sum; rows past the tile's
    // queries and chunks without a visible key leave zeros and a maximum of -inf.  (GROUPED: the one query is
    // row 0 of its tile; rows past the group's heads have nothing to leave.)
    if (GROUPED && r >= nvalid) return;
    float* p = part + (((size_t(blockIdx.x) * AQ + (GROUPED ? 0 : r)) * nq + h) * n_chunks + blockIdx.z) * (hd + 2);
#pragma unroll
    for (int i = 0; i < MAXD; ++i) {
      const int d = c16 + 16 * i;
      if (d < hd) p[d] = acc[i];
    }
    if (c16 == 0) { p[hd] = m; p[hd + 1] = l; }
    return;
  }
  if (r < nvalid) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    T* o = out + size_t(qs + q_off + (GROUPED ? 0 : r)) * (size_t(nq) * hd) + h * hd;
#pragma unroll
    for (int i = 0; i < MAXD; ++i) {
      const int d = c16 + 16 * i;
      if (d < hd) o[d] = from_float<T>(acc[i] * inv);
    }
  }
}

// Joins the chunks of one query row and head: grid (tiles * AQ rows, heads), 64 threads over the head's dimensions.
template <typename T>
__global__ __launch_bounds__(64) void attention_generic_merge_kernel(
    const float* __restrict__ part, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ tiles, T* __restrict__ out, int nq, int hd, int n_chunks) {
  const int tile = blockIdx.x / AQ, r = blockIdx.x % AQ, h = blockIdx.y;
  const int seq = tiles[2 * tile], q_off = tiles[2 * tile + 1];
  if (r >= q_len[seq] - q_off) return;
  const float* p = part + ((size_t(blockIdx.x) * nq + h) * n_chunks) * (hd + 2);
  float m = -INFINITY;
  for (int c = 0; c < n_chunks; ++c) m = fmaxf(m, p[size_t(c) * (hd + 2) + hd]);
  float l = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const float mc = p[size_t(c) * (hd + 2) + hd];
    if (mc != -INFINITY) l += expf(mc - m) * p[size_t(c) * (hd + 2) + hd + 1];
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  T* o = out + size_t(q_start[seq] + q_off + r) * (size_t(nq) * hd) + h * hd;
  for (int d = threadIdx.x; d < hd; d += 64) {
    float sum = 0.f;
    for (int c = 0; c < n_chunks; ++c) {
      const float mc = p[size_t(c) * (hd + 2) + hd];
      if (mc != -INFINITY) sum = fmaf(expf(mc - m), p[size_t(c) * (hd + 2) + d], sum);
    }
    o[d] = from_float<T>(sum * inv);
  }
}

bool attention_f32_decode_takes(int hd, int page_size, int nq, int nkv);
size_t attention_f32_decode_workspace_floats(int n_tiles, int nq, int hd, int max_ctx);
int attention_f32_decode(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                         const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* ctx_len,
                         const int32_t* tiles, int n_tiles, void* out, int nq, int nkv, int hd, int page_size,
                         int num_pages, int window, float scale, int max_ctx, float* workspace);

int attention_f32_tiles(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                        const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* q_len,
                        const int32_t* ctx_len, const int32_t* tiles, int n_tiles, void* out, int nq, int nkv, int hd,
                        int page_size, int num_pages, int window, float scale);

// Float32 storage goes to the matrix-core kernels of attention_f32.hip where they take the sizes: a step of
// one-query sequences to the one that shares a sequence's keys out over blocks, any other to the one that walks
// tiles of 32 queries.
bool attention_generic_on_matrix_cores(int dtype, int nq, int nkv, int hd, int page_size) {
  return dtype == kF32 && attention_f32_decode_takes(hd, page_size, nq, nkv);
}
static bool f32_one_query(int dtype, bool single, int nq, int nkv, int hd, int page_size) {
  return single && attention_generic_on_matrix_cores(dtype, nq, nkv, hd, page_size);
}
// Queries in a tile of the tile list that the kernels of this path expect.
int attention_generic_tile_q(int dtype, int nq, int nkv, int hd, int page_size) {
  return attention_generic_on_matrix_cores(dtype, nq, nkv, hd, page_size) ? 32 : AQ;
}

// How the keys of a step are shared out: {chunks, keys per chunk}.  One chunk unless the step has few blocks
// and long contexts; at most 32 chunks of at least 256 keys, whole groups of 32 keys each.
static void generic_chunks(int n_tiles, int rows_of_blocks, int max_tile_ctx, int* n_chunks, int* chunk) {
  *n_chunks = 1;
  *chunk = 0;
  if (n_tiles * rows_of_blocks >= 1024 || max_tile_ctx < 512) return;
  const int keys = max(256, ((max_tile_ctx + 31) / 32 + AK - 1) / AK * AK);
  *chunk = keys;
  *n_chunks = (max_tile_ctx + keys - 1) / keys;
}

// Whether a step in which every sequence brings one query (`single`) takes the grouped form of the kernel.
static bool generic_grouped(bool single, int nq, int nkv) { return single && nkv > 0 && nq % nkv == 0 && nq / nkv > 1 && nq / nkv <= AQ; }

size_t attention_generic_workspace_floats(int dtype, int page_size, int n_tiles, int nq, int nkv, int hd, int max_tile_ctx,
                                          bool single) {
  if (f32_one_query(dtype, single, nq, nkv, hd, page_size)) return attention_f32_decode_workspace_floats(n_tiles, nq, hd, max_tile_ctx);
  if (attention_generic_on_matrix_cores(dtype, nq, nkv, hd, page_size)) return 0;
  int n_chunks, chunk;
  generic_chunks(n_tiles, generic_grouped(single, nq, nkv) ? nkv : nq, max_tile_ctx, &n_chunks, &chunk);
  return n_chunks > 1 ? size_t(n_tiles) * AQ * nq * n_chunks * (hd + 2) : 0;
}

template <typename T>
int launch_attention_generic(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                             const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                             const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles,
                             void* out, int nq, int nkv, int hd, int page_size, int num_pages, int window,
                             float scale, int max_tile_ctx, float* workspace, bool single) {
  const size_t lds = sizeof(float) * (size_t(AQ + AK) * (hd + 1) + AQ * (AK + 1));
  const bool grouped = generic_grouped(single, nq, nkv);
  int n_chunks, chunk;
  generic_chunks(n_tiles, grouped ? nkv : nq, max_tile_ctx, &n_chunks, &chunk);
  if (!workspace) n_chunks = 1;
  dim3 grid(n_tiles, grouped ? nkv : nq, n_chunks);
#define SP_ATT(MAXD)                                                                                           \
  if (grouped)                                                                                                 \
    attention_generic_kernel<T, MAXD, true><<<grid, 256, lds, s>>>(                                            \
        (const T*)q, q_stride, (const T*)k_pool, (const T*)v_pool, block_tables, max_blocks, q_start, q_len,  \
        ctx_len, tiles, (T*)out, nq, nkv, hd, page_size, num_pages, window, scale, workspace, chunk);         \
  else                                                                                                         \
    attention_generic_kernel<T, MAXD, false><<<grid, 256, lds, s>>>(                                           \
        (const T*)q, q_stride, (const T*)k_pool, (const T*)v_pool, block_tables, max_blocks, q_start, q_len,  \
        ctx_len, tiles, (T*)out, nq, nkv, hd, page_size, num_pages, window, scale, workspace, chunk)
  if (hd <= 64) { SP_ATT(4); }
  else if (hd <= 128) { SP_ATT(8); }
  else if (hd <= 256) { SP_ATT(16); }
  else {
    // head sizes up to 512: the tiles of queries, keys and probabilities need more LDS than a kernel gets unasked
    static bool raised = false;
    if (!raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_generic_kernel<T, 32, true>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 112 * 1024);
      if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_generic_kernel<T, 32, false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 112 * 1024);
      if (e != hipSuccess) {
        set_error("sp_attention (generic): cannot raise the LDS limit: %s", hipGetErrorString(e));
        return 1;
      }
      raised = true;
    }
    SP_ATT(32);
  }
#undef SP_ATT
  if (check_launch("sp_attention (generic)")) return 1;
  if (n_chunks == 1) return 0;
  attention_generic_merge_kernel<T><<<dim3(n_tiles * AQ, nq), 64, 0, s>>>(workspace, q_start, q_len, tiles, (T*)out, nq, hd,
                                                                          n_chunks);
  return check_launch("sp_attention (generic, merge)");
}

int attention_generic(hipStream_t s, int dtype, const void* q, int q_stride, const void* k_pool,
                      const void* v_pool, const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                      const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles, void* out,
                      int nq, int nkv, int hd, int page_size, int num_pages, int window, float scale, int max_tile_ctx,
                      float* workspace, bool single) {
  SP_REQUIRE(int64_t(max_blocks) * page_size < (int64_t(1) << 24),
             "sp_attention: block tables of %d pages of %d tokens exceed the 2^24 positions this kernel counts",
             max_blocks, page_size);
  if (f32_one_query(dtype, single, nq, nkv, hd, page_size))
    return attention_f32_decode(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, ctx_len, tiles, n_tiles,
                                out, nq, nkv, hd, page_size, num_pages, window, scale, max_tile_ctx, workspace);
  if (attention_generic_on_matrix_cores(dtype, nq, nkv, hd, page_size))
    return attention_f32_tiles(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, q_len, ctx_len, tiles,
                               n_tiles, out, nq, nkv, hd, page_size, num_pages, window, scale);
  if (dtype == kF32)
    return launch_attention_generic<float>(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start,
                                           q_len, ctx_len, tiles, n_tiles, out, nq, nkv, hd, page_size,
                                           num_pages, window, scale, max_tile_ctx, workspace, single);
  return launch_attention_generic<bf16_t>(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start,
                                          q_len, ctx_len, tiles, n_tiles, out, nq, nkv, hd, page_size, num_pages,
                                          window, scale, max_tile_ctx, workspace, single);
}

}  // namespace sprout
