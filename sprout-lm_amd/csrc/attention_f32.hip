// One-query attention over paged float32 keys and values on the matrix cores, true 32-bit arithmetic
// (v_mfma_f32_16x16x4_f32 multiplies float32 operands and sums in float32: no reduced-precision mode).
// For steps in which every sequence brings one query (decoding) on the float32 path.
//
// One block per (256 keys, key/value head, sequence); the rows of the matrix products are the query heads of the
// group (up to 16), so a group's keys and values are read once.  Each of the four waves takes 64 keys, 16 at a time:
//   S^T[key, head]  = K[key, :] . Q[head, :]          A = 16 key rows (a lane loads 16 bytes: 4 dims), B = Q
//   O^T[dim, head] += V^T[dim, key] . P^T[key, head]   A = V^T (values lie [dim][slot] in a page), B = P
// A lane's four loaded numbers feed four successive MFMAs (k-slot l / 16 of MFMA e is dimension 4 (l / 16) + e of
// the 16 that a load covers, for both operands), and the result layout of S^T (four consecutive keys a lane) is
// the B layout of P^T under the same numbering, so probabilities never leave registers.  Softmax statistics are
// float32; the waves are merged in LDS and the blocks of a sequence by a second kernel.  Keys are cut at multiples
// of 256, 64 and 16 whatever the batch, so a position's sums do not depend on what else is in the step.
// Needs head sizes in multiples of 16 (up to 256), pages of a multiple of 4 tokens and groups of up to 16 heads;
// everything else stays with the general kernel.
#include "mfma.h"
#include "sprout_hip.h"

namespace sprout {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNoKey = -1.0e30f;      // running maximum before any key: finite, so that no inf - inf arises
constexpr int kChunk = 256, kWaveKeys = 64, kStep = 16;

__device__ __forceinline__ floatx4 mfma4(float a, float b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float max_over_quarters(float x) {   // lanes l, l ^ 16, l ^ 32, l ^ 48
  x = fmaxf(x, __shfl_xor(x, 16, 64));
  return fmaxf(x, __shfl_xor(x, 32, 64));
}

// Quotient and remainder by the page size (known at launch only) for 0 <= x < 2^24: a float product and one
// step of correction either way, instead of the long sequence of an integer division.
struct PageDivider {
  int d;
  float inv;
  __device__ __forceinline__ void divmod(int x, int& q, int& r) const {
    q = int(float(x) * inv);
    r = x - q * d;
    if (r < 0) { r += d; --q; }
    if (r >= d) { r -= d; ++q; }
  }
};

template <int DT, int SB>   // head size 16 DT; SB steps of 16 keys are requested together
__global__ __launch_bounds__(256) void attention_f32_decode_kernel(
    const float* __restrict__ q, int q_stride, const float* __restrict__ k_pool, const float* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ tiles, float* __restrict__ out,
    float* __restrict__ part_o, float* __restrict__ part_ml, int n_splits, int nq, int nkv, int page_size,
    int num_pages, int window, float scale2) {
  constexpr int HD = 16 * DT;
  extern __shared__ float f32_lds[];
  float* s_o = f32_lds;                                   // [4][16][HD + 1]
  float* s_m = s_o + 4 * 16 * (HD + 1);                   // [4][16]
  float* s_l = s_m + 64;                                  // [4][16]
  int32_t* s_table = reinterpret_cast<int32_t*>(s_l + 64);  // the chunk's page numbers: up to 256 / 4 + 1
  const int split = blockIdx.x, g = blockIdx.y, ti = blockIdx.z;
  const int seq = tiles[2 * ti];
  const int chunk0 = split * kChunk;
  PageDivider by_page;
  by_page.d = page_size;
  by_page.inv = 1.0f / float(page_size);
  int table_first, table_last, unused;
  by_page.divmod(chunk0, table_first, unused);
  by_page.divmod(chunk0 + kChunk - 1, table_last, unused);
  if (int(threadIdx.x) <= table_last - table_first)
    s_table[threadIdx.x] = block_tables[size_t(seq) * max_blocks + min(table_first + int(threadIdx.x), max_blocks - 1)];
  const int q_row = q_start[seq];
  const int ctx = ctx_len[seq], pos = ctx - 1;
  const int k_lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int G = nq / nkv;
  if (chunk0 > pos || chunk0 + kChunk <= k_lo) {
    // no visible key in this chunk: the merge reads every chunk's (maximum, sum), so an empty chunk says so itself
    if (n_splits > 1 && int(threadIdx.x) < G) {
      const size_t slot = (size_t(ti) * nq + g * G + threadIdx.x) * n_splits + split;
      part_ml[2 * slot] = kNoKey;
      part_ml[2 * slot + 1] = 0.f;
    }
    return;
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  const size_t page_stride = size_t(nkv) * page_size * HD;
  const float* kbase = k_pool + size_t(g) * page_size * HD;
  const float* vbase = v_pool + size_t(g) * page_size * HD;

  float4 qv[DT];
#pragma unroll
  for (int c = 0; c < DT; ++c)
    qv[c] = lr < G ? *reinterpret_cast<const float4*>(q + size_t(q_row) * q_stride + (g * G + lr) * HD + 16 * c + 4 * lj)
                   : make_float4(0.f, 0.f, 0.f, 0.f);
  __syncthreads();   // the page numbers are in LDS

  floatx4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = kNoKey, lsum = 0.f;
  const int w0 = chunk0 + wave * kWaveKeys;

#pragma unroll
  for (int b = 0; b < kWaveKeys / kStep; b += SB) {
    float4 kr[SB][DT], vr[SB][DT];
    bool live[SB];
#pragma unroll
    for (int i = 0; i < SB; ++i) {
      const int key0 = w0 + kStep * (b + i);
      live[i] = key0 <= pos && key0 + kStep > k_lo;      // the same in every lane of the wave
      if (!live[i]) continue;
      // loads are clamped to the visible keys; what lies outside is masked by position below
      int logical, slot;
      by_page.divmod(min(max(key0 + lr, k_lo), pos), logical, slot);
      int page = min(max(s_table[logical - table_first], 0), num_pages - 1);   // a bad entry must not become a wild address
      const float* krow = kbase + size_t(page) * page_stride + size_t(slot) * HD + 4 * lj;
#pragma unroll
      for (int c = 0; c < DT; ++c) kr[i][c] = *reinterpret_cast<const float4*>(krow + 16 * c);
      by_page.divmod(min(max(key0 + 4 * lj, (k_lo >> 2) << 2), (pos >> 2) << 2), logical, slot);
      page = min(max(s_table[logical - table_first], 0), num_pages - 1);
      const float* vcol = vbase + size_t(page) * page_stride + slot + size_t(lr) * page_size;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vr[i][dt] = *reinterpret_cast<const float4*>(vcol + size_t(16 * dt) * page_size);
    }
#pragma unroll
    for (int i = 0; i < SB; ++i) {
      if (!live[i]) continue;
      const int key0 = w0 + kStep * (b + i);
      floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DT; ++c) {
        s = mfma4(kr[i][c].x, qv[c].x, s);
        s = mfma4(kr[i][c].y, qv[c].y, s);
        s = mfma4(kr[i][c].z, qv[c].z, s);
        s = mfma4(kr[i][c].w, qv[c].w, s);
      }
      // element e of s: key key0 + 4 lj + e, head lr
      float sv[4], top = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + 4 * lj + e;
        sv[e] = (key >= k_lo && key <= pos) ? s[e] * scale2 : -INFINITY;
        top = fmaxf(top, sv[e]);
      }
      top = max_over_quarters(top);
      const float m_new = fmaxf(m, top);            // finite: m starts finite
      const float alpha = exp2f(m - m_new);
      m = m_new;
      lsum *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] *= alpha;
      float p[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        p[e] = exp2f(sv[e] - m);                    // exp2(-inf) = 0 for masked keys
        lsum += p[e];
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        o[dt] = mfma4(vr[i][dt].x, p[0], o[dt]);
        o[dt] = mfma4(vr[i][dt].y, p[1], o[dt]);
        o[dt] = mfma4(vr[i][dt].z, p[2], o[dt]);
        o[dt] = mfma4(vr[i][dt].w, p[3], o[dt]);
      }
    }
  }
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);
  if (lj == 0) { s_m[wave * 16 + lr] = m; s_l[wave * 16 + lr] = lsum; }
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int e = 0; e < 4; ++e) s_o[(wave * 16 + lr) * (HD + 1) + 16 * dt + 4 * lj + e] = o[dt][e];
  __syncthreads();

  for (int i = threadIdx.x; i < G * HD; i += 256) {
    const int qh = i / HD, d = i % HD;
    float mx = s_m[qh];
#pragma unroll
    for (int w = 1; w < 4; ++w) mx = fmaxf(mx, s_m[w * 16 + qh]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = exp2f(s_m[w * 16 + qh] - mx);
      num = fmaf(f, s_o[(w * 16 + qh) * (HD + 1) + d], num);
      den = fmaf(f, s_l[w * 16 + qh], den);
    }
    const int head = g * G + qh;
    if (n_splits == 1) {
      out[size_t(q_row) * (size_t(nq) * HD) + head * HD + d] = den > 0.f ? num / den : 0.f;
    } else {
      const size_t slot = (size_t(ti) * nq + head) * n_splits + split;
      part_o[slot * HD + d] = num;
      if (d == 0) { part_ml[2 * slot] = mx; part_ml[2 * slot + 1] = den; }
    }
  }
}

// Joins the chunks of one (sequence, head), in the order of the chunks: grid (sequences, heads), one wave.  What a
// lane reads depends on its indices alone (empty chunks say so themselves), so it asks for 16 chunks at a time.
__global__ __launch_bounds__(64) void attention_f32_merge_kernel(const float* __restrict__ part_o,
                                                                 const float* __restrict__ part_ml,
                                                                 const int32_t* __restrict__ q_start,
                                                                 const int32_t* __restrict__ tiles,
                                                                 float* __restrict__ out, int n_splits, int nq, int hd) {
  constexpr int GROUP = 16;
  const int ti = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int seq = tiles[2 * ti];
  const size_t base = (size_t(ti) * nq + head) * n_splits;
  float mx = kNoKey, den = 0.f, num[4] = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = 0; s0 < n_splits; s0 += GROUP) {
    float ms[GROUP], ls[GROUP], os[GROUP][4];
#pragma unroll
    for (int i = 0; i < GROUP; ++i) {
      const bool in = s0 + i < n_splits;
      ms[i] = in ? part_ml[2 * (base + s0 + i)] : kNoKey;
      ls[i] = in ? part_ml[2 * (base + s0 + i) + 1] : 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        os[i][j] = (in && d < hd) ? part_o[(base + s0 + i) * hd + d] : 0.f;
      }
    }
    float top = mx;
#pragma unroll
    for (int i = 0; i < GROUP; ++i) top = fmaxf(top, ms[i]);
    const float keep = exp2f(mx - top);
    mx = top;
    den *= keep;
#pragma unroll
    for (int j = 0; j < 4; ++j) num[j] *= keep;
#pragma unroll
    for (int i = 0; i < GROUP; ++i) {
      if (ls[i] > 0.f) {                      // an empty chunk left nothing to read in part_o
        const float f = exp2f(ms[i] - mx);
        den = fmaf(f, ls[i], den);
#pragma unroll
        for (int j = 0; j < 4; ++j) num[j] = fmaf(f, os[i][j], num[j]);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int d = lane + 64 * j;
    if (d < hd) out[size_t(q_start[seq]) * (size_t(nq) * hd) + head * hd + d] = den > 0.f ? num[j] / den : 0.f;
  }
}

// ------------------------------------------------------------------------------------------------ several queries
// Steps with portions of prompts: one block per (tile of 32 queries of a sequence, up to four query heads of one
// key/value head), one wave per head, so the waves of a block walk the same keys at the same time and fetch them
// once between them (the second wave on finds them in the CU's cache) and every wave has a SIMD of its own: the
// matrix cores bound this kernel, and a prompt's last tile, which walks every key, bounds the launch.  Tiles are
// taken from the end of the list, the longest walks first.  A wave holds two tiles of 16 queries as the B operands
//   S^T[key, query] = K[key, :] . Q[query, :]       O^T[dim, query] += V^T[dim, key] . P^T[key, query]
// and walks the keys 16 at a time from a multiple of 16, the next step's keys and values requested while the
// current ones are multiplied (head sizes up to 64; above that the registers do not hold two steps).  Causal
// mask and window by position; softmax statistics float32.  A sequence with one query is a tile with one row.
// MAXW: the most waves (query heads of a group) a block may have; it sets the registers a wave may use.
template <int DT, bool AHEAD, int MAXW>
__global__ __launch_bounds__(64 * MAXW) void attention_f32_tiles_kernel(
    const float* __restrict__ q, int q_stride, const float* __restrict__ k_pool, const float* __restrict__ v_pool,
    const int32_t* __restrict__ block_tables, int max_blocks, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ q_len, const int32_t* __restrict__ ctx_len, const int32_t* __restrict__ tiles,
    float* __restrict__ out, int nq, int nkv, int page_size, int num_pages, int window, float scale2) {
  constexpr int HD = 16 * DT;
  const int tile = gridDim.x - 1 - blockIdx.x;
  const int seq = tiles[2 * tile], q_off = tiles[2 * tile + 1];
  const int G = nq / nkv, parts = (G + MAXW - 1) / MAXW;      // a group's heads in `parts` blocks of up to MAXW
  const int g = blockIdx.y / parts, part = blockIdx.y % parts;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lj = lane >> 4;
  if (part * MAXW + wave >= G) return;
  const int head = g * G + part * MAXW + wave;
  const int qlen = q_len[seq], ctx = ctx_len[seq], qs = q_start[seq];
  const int nvalid = min(32, qlen - q_off);
  if (nvalid <= 0) return;
  const int pos0 = ctx - qlen + q_off;                 // position of the tile's first query
  const int last_pos = pos0 + nvalid - 1;
  const int32_t* table = block_tables + size_t(seq) * max_blocks;
  PageDivider by_page;
  by_page.d = page_size;
  by_page.inv = 1.0f / float(page_size);
  const size_t page_stride = size_t(nkv) * page_size * HD;
  const float* kbase = k_pool + size_t(g) * page_size * HD;
  const float* vbase = v_pool + size_t(g) * page_size * HD;

  float4 qv[2][DT];
  int qpos[2];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    const int row = 16 * qt + lr;
    qpos[qt] = row < nvalid ? pos0 + row : -1;
#pragma unroll
    for (int c = 0; c < DT; ++c)
      qv[qt][c] = row < nvalid ? *reinterpret_cast<const float4*>(q + size_t(qs + q_off + row) * q_stride + head * HD + 16 * c + 4 * lj)
                               : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  floatx4 o[2][DT];
  float m[2] = {kNoKey, kNoKey}, lsum[2] = {0.f, 0.f};
#pragma unroll
  for (int qt = 0; qt < 2; ++qt)
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[qt][dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int k_lo = window > 0 ? max(0, pos0 - window + 1) : 0;     // the oldest key any query of the tile sees
  const int first_key = (k_lo / kStep) * kStep;

  auto load = [&](int key0, float4 (&kr)[DT], float4 (&vr)[DT]) {
    int logical, slot;
    by_page.divmod(min(max(key0 + lr, k_lo), last_pos), logical, slot);
    int page = min(max(table[min(logical, max_blocks - 1)], 0), num_pages - 1);
    const float* krow = kbase + size_t(page) * page_stride + size_t(slot) * HD + 4 * lj;
#pragma unroll
    for (int c = 0; c < DT; ++c) kr[c] = *reinterpret_cast<const float4*>(krow + 16 * c);
    by_page.divmod(min(max(key0 + 4 * lj, (k_lo >> 2) << 2), (last_pos >> 2) << 2), logical, slot);
    page = min(max(table[min(logical, max_blocks - 1)], 0), num_pages - 1);
    const float* vcol = vbase + size_t(page) * page_stride + slot + size_t(lr) * page_size;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vr[dt] = *reinterpret_cast<const float4*>(vcol + size_t(16 * dt) * page_size);
  };
  auto attend = [&](int key0, const float4 (&kr)[DT], const float4 (&vr)[DT]) {
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      if (qt == 1 && nvalid <= 16) break;              // the same in every lane
      floatx4 s = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DT; ++c) {
        s = mfma4(kr[c].x, qv[qt][c].x, s);
        s = mfma4(kr[c].y, qv[qt][c].y, s);
        s = mfma4(kr[c].z, qv[qt][c].z, s);
        s = mfma4(kr[c].w, qv[qt][c].w, s);
      }
      const int hi = qpos[qt], lo = window > 0 ? max(0, hi - window + 1) : 0;
      float sv[4], top = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int key = key0 + 4 * lj + e;
        sv[e] = (key >= lo && key <= hi) ? s[e] * scale2 : -INFINITY;      // hi = -1: a row that does not exist
        top = fmaxf(top, sv[e]);
      }
      top = max_over_quarters(top);
      const float m_new = fmaxf(m[qt], top);
      const float alpha = exp2f(m[qt] - m_new);
      m[qt] = m_new;
      lsum[qt] *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[qt][dt] *= alpha;
      float p[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        p[e] = exp2f(sv[e] - m_new);
        lsum[qt] += p[e];
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        o[qt][dt] = mfma4(vr[dt].x, p[0], o[qt][dt]);
        o[qt][dt] = mfma4(vr[dt].y, p[1], o[qt][dt]);
        o[qt][dt] = mfma4(vr[dt].z, p[2], o[qt][dt]);
        o[qt][dt] = mfma4(vr[dt].w, p[3], o[qt][dt]);
      }
    }
  };

  if (AHEAD) {
    float4 ka[DT], va[DT], kb[DT], vb[DT];
    load(first_key, ka, va);
    for (int key0 = first_key; key0 <= last_pos; key0 += 2 * kStep) {
      const bool second = key0 + kStep <= last_pos;
      if (second) load(key0 + kStep, kb, vb);
      attend(key0, ka, va);
      if (!second) break;
      if (key0 + 2 * kStep <= last_pos) load(key0 + 2 * kStep, ka, va);
      attend(key0 + kStep, kb, vb);
    }
  } else {
    float4 ka[DT], va[DT];
    for (int key0 = first_key; key0 <= last_pos; key0 += kStep) {
      load(key0, ka, va);
      attend(key0, ka, va);
    }
  }
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    float l = lsum[qt];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const int row = 16 * qt + lr;
    if (row >= nvalid) continue;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float* dst = out + size_t(qs + q_off + row) * (size_t(nq) * HD) + head * HD + 4 * lj;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      *reinterpret_cast<float4*>(dst + 16 * dt) = make_float4(o[qt][dt][0] * inv, o[qt][dt][1] * inv, o[qt][dt][2] * inv, o[qt][dt][3] * inv);
  }
}

template <int DT>
int launch_tiles(hipStream_t s, const float* q, int q_stride, const float* k_pool, const float* v_pool,
                 const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* q_len,
                 const int32_t* ctx_len, const int32_t* tiles, int n_tiles, float* out, int nq, int nkv, int page_size,
                 int num_pages, int window, float scale) {
  const int G = nq / nkv, parts = (G + 3) / 4;
  attention_f32_tiles_kernel<DT, (DT <= 8), 4><<<dim3(n_tiles, nkv * parts), 64 * min(G, 4), 0, s>>>(
      q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, q_len, ctx_len, tiles, out, nq, nkv, page_size,
      num_pages, window, scale * kLog2e);
  return check_launch("sp_attention (float32, tiles)");
}

size_t decode_lds_bytes(int hd) { return sizeof(float) * (size_t(4) * 16 * (hd + 1) + 128) + sizeof(int32_t) * (kChunk / 4 + 4); }

template <int DT, int SB>
int launch_decode(hipStream_t s, const float* q, int q_stride, const float* k_pool, const float* v_pool,
                  const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* ctx_len,
                  const int32_t* tiles, int n_tiles, float* out, float* workspace, int n_splits, int nq, int nkv,
                  int page_size, int num_pages, int window, float scale) {
  constexpr int HD = 16 * DT;
  const size_t lds = decode_lds_bytes(HD);
  static bool raised = false;
  if (lds > 48 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_f32_decode_kernel<DT, SB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (e != hipSuccess) {
      set_error("sp_attention (float32, one query): cannot raise the LDS limit: %s", hipGetErrorString(e));
      return 1;
    }
    raised = true;
  }
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + size_t(n_tiles) * nq * n_splits * HD : nullptr;
  attention_f32_decode_kernel<DT, SB><<<dim3(n_splits, nkv, n_tiles), 256, lds, s>>>(
      q, q_stride, k_pool, v_pool, block_tables, max_blocks, q_start, ctx_len, tiles, out, part_o, part_ml, n_splits,
      nq, nkv, page_size, num_pages, window, scale * kLog2e);
  if (check_launch("sp_attention (float32, one query)")) return 1;
  if (n_splits == 1) return 0;
  attention_f32_merge_kernel<<<dim3(n_tiles, nq), 64, 0, s>>>(part_o, part_ml, q_start, tiles, out, n_splits, nq, HD);
  return check_launch("sp_attention (float32, one query, merge)");
}

}  // namespace

// Whether the kernel of this file takes a step of one-query sequences with these sizes.
bool attention_f32_decode_takes(int hd, int page_size, int nq, int nkv) {
  return hd > 0 && hd <= 256 && hd % 16 == 0 && page_size > 0 && page_size % 4 == 0 && nkv > 0 && nq % nkv == 0 &&
         nq / nkv <= 16;
}

static int f32_splits(int max_ctx) { return max_ctx > 0 ? (max_ctx + kChunk - 1) / kChunk : 1; }

size_t attention_f32_decode_workspace_floats(int n_tiles, int nq, int hd, int max_ctx) {
  const int n = f32_splits(max_ctx);
  return n > 1 ? size_t(n_tiles) * nq * n * (hd + 2) : 0;
}

int attention_f32_decode(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                         const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* ctx_len,
                         const int32_t* tiles, int n_tiles, void* out, int nq, int nkv, int hd, int page_size,
                         int num_pages, int window, float scale, int max_ctx, float* workspace) {
  SP_REQUIRE(attention_f32_decode_takes(hd, page_size, nq, nkv), "sp_attention (float32, one query): sizes not taken");
  SP_REQUIRE(max_ctx <= max_blocks * page_size, "sp_attention: a context of %d tokens exceeds the block tables (%d pages of %d)",
             max_ctx, max_blocks, page_size);
  SP_REQUIRE((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool)) % 16 == 0 &&
                 q_stride % 4 == 0,
             "sp_attention (float32, one query): operands must be 16-byte aligned");
  const int n_splits = f32_splits(max_ctx);
  SP_REQUIRE(n_splits == 1 || workspace, "sp_attention (float32, one query): missing workspace");
#define SP_F32_DECODE(DT, SB)                                                                                     \
  return launch_decode<DT, SB>(s, (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool,          \
                               block_tables, max_blocks, q_start, ctx_len, tiles, n_tiles, (float*)out, workspace, \
                               n_splits, nq, nkv, page_size, num_pages, window, scale)
  switch (hd / 16) {
    case 1: SP_F32_DECODE(1, 4);
    case 2: SP_F32_DECODE(2, 4);
    case 3: SP_F32_DECODE(3, 4);
    case 4: SP_F32_DECODE(4, 4);
    case 5: SP_F32_DECODE(5, 2);
    case 6: SP_F32_DECODE(6, 2);
    case 7: SP_F32_DECODE(7, 2);
    case 8: SP_F32_DECODE(8, 2);
    case 9: SP_F32_DECODE(9, 1);
    case 10: SP_F32_DECODE(10, 1);
    case 11: SP_F32_DECODE(11, 1);
    case 12: SP_F32_DECODE(12, 1);
    case 13: SP_F32_DECODE(13, 1);
    case 14: SP_F32_DECODE(14, 1);
    case 15: SP_F32_DECODE(15, 1);
    default: SP_F32_DECODE(16, 1);
  }
#undef SP_F32_DECODE
}

int attention_f32_tiles(hipStream_t s, const void* q, int q_stride, const void* k_pool, const void* v_pool,
                        const int32_t* block_tables, int max_blocks, const int32_t* q_start, const int32_t* q_len,
                        const int32_t* ctx_len, const int32_t* tiles, int n_tiles, void* out, int nq, int nkv, int hd,
                        int page_size, int num_pages, int window, float scale) {
  SP_REQUIRE(attention_f32_decode_takes(hd, page_size, nq, nkv), "sp_attention (float32, tiles): sizes not taken");
  SP_REQUIRE((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(k_pool) | reinterpret_cast<uintptr_t>(v_pool) |
              reinterpret_cast<uintptr_t>(out)) % 16 == 0 && q_stride % 4 == 0,
             "sp_attention (float32, tiles): operands must be 16-byte aligned");
#define SP_F32_TILES(DT)                                                                                          \
  case DT:                                                                                                        \
    return launch_tiles<DT>(s, (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool, block_tables, \
                            max_blocks, q_start, q_len, ctx_len, tiles, n_tiles, (float*)out, nq, nkv, page_size,  \
                            num_pages, window, scale)
  switch (hd / 16) {
    SP_F32_TILES(1); SP_F32_TILES(2); SP_F32_TILES(3); SP_F32_TILES(4); SP_F32_TILES(5); SP_F32_TILES(6);
    SP_F32_TILES(7); SP_F32_TILES(8); SP_F32_TILES(9); SP_F32_TILES(10); SP_F32_TILES(11); SP_F32_TILES(12);
    SP_F32_TILES(13); SP_F32_TILES(14); SP_F32_TILES(15);
    default: return launch_tiles<16>(s, (const float*)q, q_stride, (const float*)k_pool, (const float*)v_pool,
                                     block_tables, max_blocks, q_start, q_len, ctx_len, tiles, n_tiles, (float*)out, nq,
                                     nkv, page_size, num_pages, window, scale);
  }
#undef SP_F32_TILES
}

}  // namespace sprout
