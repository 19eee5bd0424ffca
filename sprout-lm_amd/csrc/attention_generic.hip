// Causal grouped-query attention of a mixed batch over paged keys and values, float32 arithmetic.
// Any head size up to 256, any page size, any number of heads and groups, optional window.
// One block works on 16 queries of one sequence and one head, walking the keys 32 at a time with a
// running maximum and sum (all float32).  Keys are always walked from a multiple of 32, so the order
// of the sums at a position does not depend on how the tokens were cut into steps.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

constexpr int AQ = 16;  // queries per block
constexpr int AK = 32;  // keys per iteration

template <typename T, int MAXD>  // MAXD = ceil(hd / 16) upper bound
__global__ __launch_bounds__(256) void attention_generic_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ k_pool, const T* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ tiles,
    T* __restrict__ out, int nq, int nkv, int hd, int page_size, int num_pages, int window, float scale) {
  extern __shared__ float lds[];
  float* Qs = lds;                         // [AQ][hd]
  float* KVs = Qs + AQ * hd;               // [AK][hd + 1]
  float* Ps = KVs + AK * (hd + 1);         // [AQ][AK]
  const int kv_stride = hd + 1;

  const int seq = tiles[2 * blockIdx.x], q_off = tiles[2 * blockIdx.x + 1];
  const int h = blockIdx.y;
  const int qlen = q_len[seq], ctx = ctx_len[seq], qs = q_start[seq];
  const int nvalid = min(AQ, qlen - q_off);
  if (nvalid <= 0) return;
  const int pos0 = ctx - qlen + q_off;
  const int g = h / (nq / nkv);
  const int32_t* bt = block_tables + size_t(seq) * max_blocks;

  for (int i = threadIdx.x; i < AQ * hd; i += 256) {
    const int r = i / hd, d = i % hd;
    Qs[i] = r < nvalid ? to_float(q[size_t(qs + q_off + r) * q_stride + h * hd + d]) : 0.f;
  }

  const int r = threadIdx.x / 16, c16 = threadIdx.x % 16;
  const int my_pos = pos0 + r;
  const int k_end = pos0 + nvalid;  // one past the last visible key of the tile
  const int k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) acc[i] = 0.f;

  for (int kb = (k_lo / AK) * AK; kb < k_end; kb += AK) {
    __syncthreads();  // Qs written / previous V tile consumed
    for (int i = threadIdx.x; i < AK * hd; i += 256) {
      const int jj = i / hd, d = i % hd, j = kb + jj;
      float v = 0.f;
      if (j >= k_lo && j < k_end) {
        const int page = bt[j / page_size];
        if (page >= 0 && page < num_pages)
          v = to_float(k_pool[((size_t(page) * nkv + g) * page_size + j % page_size) * hd + d]);
      }
      KVs[jj * kv_stride + d] = v;
    }
    __syncthreads();
    float s[2];
    float row_max = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int c = c16 + 16 * u, j = kb + c;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(Qs[r * hd + d], KVs[c * kv_stride + d], dot);
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
    Ps[r * AK + c16] = p[0];
    Ps[r * AK + c16 + 16] = p[1];
    __syncthreads();  // scores done with the K tile; Ps complete
    for (int i = threadIdx.x; i < AK * hd; i += 256) {
      const int jj = i / hd, d = i % hd, j = kb + jj;
      float v = 0.f;
      if (j >= k_lo && j < k_end) {
        const int page = bt[j / page_size];
        if (page >= 0 && page < num_pages)
          v = to_float(v_pool[((size_t(page) * nkv + g) * hd + d) * page_size + j % page_size]);
      }
      KVs[jj * kv_stride + d] = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MAXD; ++i) {
      const int d = c16 + 16 * i;
      if (d < hd) {
        float sum = acc[i] * alpha;
        for (int c = 0; c < AK; ++c) sum = fmaf(Ps[r * AK + c], KVs[c * kv_stride + d], sum);
        acc[i] = sum;
      }
    }
  }
  if (r < nvalid) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    T* o = out + size_t(qs + q_off + r) * (size_t(nq) * hd) + h * hd;
#pragma unroll
    for (int i = 0; i < MAXD; ++i) {
      const int d = c16 + 16 * i;
      if (d < hd) o[d] = from_float<T>(acc[i] * inv);
    }
  }
}

template <typename T>
int launch_attention_generic(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                             const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                             const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles,
                             void* out, int nq, int nkv, int hd, int page_size, int num_pages, int window,
                             float scale) {
  const size_t lds = sizeof(float) * (size_t(AQ) * hd + size_t(AK) * (hd + 1) + AQ * AK);
  dim3 grid(n_tiles, nq);
#define SP_ATT(MAXD)                                                                                        \
  attention_generic_kernel<T, MAXD><<<grid, 256, lds, s>>>(                                                 \
      (const T*)q, q_stride, (const T*)k_pool, (const T*)v_pool, block_tables, max_blocks, q_start, q_len, \
      ctx_len, tiles, (T*)out, nq, nkv, hd, page_size, num_pages, window, scale)
  if (hd <= 64) SP_ATT(4);
  else if (hd <= 128) SP_ATT(8);
  else SP_ATT(16);
#undef SP_ATT
  return check_launch("sp_attention (generic)");
}

int attention_generic(hipStream_t s, int dtype, const void* q, int q_stride, const void* k_pool,
                      const void* v_pool, const int32_t* block_tables, int max_blocks, const int32_t* q_start,
                      const int32_t* q_len, const int32_t* ctx_len, const int32_t* tiles, int n_tiles, void* out,
                      int nq, int nkv, int hd, int page_size, int num_pages, int window, float scale) {
  if (dtype == kF32)
    return launch_attention_generic<float>(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start,
                                           q_len, ctx_len, tiles, n_tiles, out, nq, nkv, hd, page_size,
                                           num_pages, window, scale);
  return launch_attention_generic<bf16_t>(s, q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start,
                                          q_len, ctx_len, tiles, n_tiles, out, nq, nkv, hd, page_size, num_pages,
                                          window, scale);
}

}  // namespace sprout
