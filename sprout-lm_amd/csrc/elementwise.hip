// Embedding gather, RMSNorm, SiLU-gated product, and rotation + cache write.
// All arithmetic is float32; only loads and stores see the storage type.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {

// ---------------------------------------------------------------- embedding
template <typename TW>
__global__ void embed_kernel(const TW* __restrict__ table, const int32_t* __restrict__ tokens,
                             float* __restrict__ residual, int H) {
  const int t = blockIdx.x;
  const TW* row = table + size_t(tokens[t]) * H;
  float* out = residual + size_t(t) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_float(row[i]);
}

// ---------------------------------------------------------------- RMSNorm
// y = (x * rsqrt(mean(x^2) + eps)) * w, the normalised value rounded to float32 before the weight.
template <typename TW, typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                               const TW* __restrict__ w, float eps, TO* __restrict__ out, int H) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* in = x + size_t(rows ? rows[r] : r) * H;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = in[i];
    sum = fmaf(v, v, sum);
  }
  sum = block_sum(sum, scratch);
  const float scale = 1.0f / sqrtf(sum / float(H) + eps);
  TO* o = out + size_t(r) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float n = in[i] * scale;
    o[i] = from_float<TO>(n * to_float(w[i]));
  }
}

// The same for rows of H = 4 n elements of at most 4 * PER * blockDim.x: a thread keeps its PER groups of four
// in registers between the sum and the scaling (one trip to memory, 16-byte loads).
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 b = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(b.x << 16), __uint_as_float(b.x & 0xffff0000u), __uint_as_float(b.y << 16),
                     __uint_as_float(b.y & 0xffff0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(uint32_t(f32_to_bf16_bits(v.x)) | (uint32_t(f32_to_bf16_bits(v.y)) << 16),
                                            uint32_t(f32_to_bf16_bits(v.z)) | (uint32_t(f32_to_bf16_bits(v.w)) << 16));
}

template <typename TW, typename TO, int PER>
__global__ void rmsnorm_rows_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                    const TW* __restrict__ w, float eps, TO* __restrict__ out, int H) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* in = x + size_t(rows ? rows[r] : r) * H;
  float4 v[PER], wv[PER];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = 4 * (threadIdx.x + j * blockDim.x);
    v[j] = i < H ? load4(in + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    wv[j] = i < H ? load4(w + i) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
#pragma unroll
  for (int j = 0; j < PER; ++j) sum = fmaf(v[j].x, v[j].x, fmaf(v[j].y, v[j].y, fmaf(v[j].z, v[j].z, fmaf(v[j].w, v[j].w, sum))));
  sum = block_sum(sum, scratch);
  const float scale = 1.0f / sqrtf(sum / float(H) + eps);
  TO* o = out + size_t(r) * H;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = 4 * (threadIdx.x + j * blockDim.x);
    if (i < H)
      store4(o + i, make_float4((v[j].x * scale) * wv[j].x, (v[j].y * scale) * wv[j].y, (v[j].z * scale) * wv[j].z,
                                (v[j].w * scale) * wv[j].w));
  }
}

// ---------------------------------------------------------------- SiLU(gate) * up
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= I) return;
  const float g = to_float(gu[size_t(t) * 2 * I + i]);
  const float u = to_float(gu[size_t(t) * 2 * I + I + i]);
  const float s = g / (1.0f + expf(-g));
  out[size_t(t) * I + i] = from_float<T>(s * u);
}

// ---------------------------------------------------------------- rotation + cache write
// One block per token.  Pair (d, d + rotary_dim/2) of each q and k head turns by
// positions[t] * inv_freq[d]; k (rotated) and v go to the pools.  Keys lie [page][group][slot][dim]; values lie
// [page][group][dim][slot], so that the keys of one dimension are contiguous for the P.V matrix product.
// inv_freq_tail (float32 storage only, may be null): what the float32 table lost of the float64 one.  With it
// the angle and its sine and cosine are computed in float64: a float32 angle is off by up to position * 6e-8,
// which at positions in the thousands is more than all other roundings of the float32 path together.
// bfloat16, head sizes and rotary sizes that are multiples of 8: a thread owns four consecutive pairs (d, d +
// rotary_dim / 2), computes their sines and cosines once and turns those pairs of every q and k head with them
// (8-byte loads and stores); then the part of k beyond rotary_dim and v go to the pools.
__global__ void rope_cache_bf16_kernel(bf16_t* __restrict__ qkv, const int32_t* __restrict__ positions,
                                       const float* __restrict__ inv_freq, int rotary_dim,
                                       const int32_t* __restrict__ slot_mapping, bf16_t* __restrict__ k_pool,
                                       bf16_t* __restrict__ v_pool, int nq, int nkv, int hd, int page_size) {
  const int t = blockIdx.x;
  const int width = (nq + 2 * nkv) * hd;
  bf16_t* row = qkv + size_t(t) * width;
  const float pos = float(positions[t]);
  const int half = rotary_dim / 2, groups = half / 4;          // groups of four pairs per head
  const int slot = nkv ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  if (groups > 0 && int(threadIdx.x) < (int(blockDim.x) / groups) * groups) {
    const int d = 4 * (threadIdx.x % groups), head0 = threadIdx.x / groups, head_step = blockDim.x / groups;
    float sn[4], cs[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) sincosf(pos * inv_freq[d + j], &sn[j], &cs[j]);
    for (int head = head0; head < nq + nkv; head += head_step) {
      bf16_t* h = row + size_t(head) * hd;
      const float4 a = load4(h + d), b = load4(h + d + half);
      const float4 ra = make_float4(a.x * cs[0] - b.x * sn[0], a.y * cs[1] - b.y * sn[1], a.z * cs[2] - b.z * sn[2],
                                    a.w * cs[3] - b.w * sn[3]);
      const float4 rb = make_float4(b.x * cs[0] + a.x * sn[0], b.y * cs[1] + a.y * sn[1], b.z * cs[2] + a.z * sn[2],
                                    b.w * cs[3] + a.w * sn[3]);
      store4(h + d, ra);
      store4(h + d + half, rb);
      if (head >= nq && slot >= 0) {
        bf16_t* dst = k_pool + ((size_t(page) * nkv + (head - nq)) * page_size + off) * hd;
        store4(dst + d, ra);
        store4(dst + d + half, rb);
      }
    }
  }
  if (slot < 0) return;
  if (rotary_dim < hd) {
    const int rest = hd - rotary_dim;
    for (int i = threadIdx.x; i < nkv * rest; i += blockDim.x) {
      const int g = i / rest, d = rotary_dim + i % rest;
      k_pool[((size_t(page) * nkv + g) * page_size + off) * hd + d] = row[size_t(nq + g) * hd + d];
    }
  }
  for (int i = threadIdx.x; i < nkv * hd / 4; i += blockDim.x) {
    const int g = (4 * i) / hd, d = (4 * i) % hd;
    const uint2 v = *reinterpret_cast<const uint2*>(row + size_t(nq + nkv + g) * hd + d);
    bf16_t* dst = v_pool + ((size_t(page) * nkv + g) * hd + d) * page_size + off;
    dst[0] = bf16_t{uint16_t(v.x & 0xffffu)};
    dst[page_size] = bf16_t{uint16_t(v.x >> 16)};
    dst[2 * size_t(page_size)] = bf16_t{uint16_t(v.y & 0xffffu)};
    dst[3 * size_t(page_size)] = bf16_t{uint16_t(v.y >> 16)};
  }
}

// (cosine, sine) of positions[t] * inv_freq[d] for every token and pair: computed once per step for all layers.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq, int half,
                                  float2* __restrict__ out, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float sn, cs;
  sincosf(float(positions[i / half]) * inv_freq[i % half], &sn, &cs);
  out[i] = make_float2(cs, sn);
}

template <typename T>
__global__ void rope_cache_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq, const float* __restrict__ inv_freq_tail, int rotary_dim,
                                  const int32_t* __restrict__ slot_mapping, T* __restrict__ k_pool,
                                  T* __restrict__ v_pool, int nq, int nkv, int hd, int page_size) {
  const int t = blockIdx.x;
  const int width = (nq + 2 * nkv) * hd;
  T* row = qkv + size_t(t) * width;
  const float pos = float(positions[t]);
  const int half = rotary_dim / 2;
  const int slot = nkv ? slot_mapping[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;

  // rotate q heads in place, k heads in place and into the pool
  const int pairs = (nq + nkv) * half;
  for (int i = threadIdx.x; i < pairs; i += blockDim.x) {
    const int head = i / half, d = i % half;
    float sn, cs;
    if (inv_freq_tail) {
      double sn64, cs64;
      sincos(double(positions[t]) * (double(inv_freq[d]) + double(inv_freq_tail[d])), &sn64, &cs64);
      sn = float(sn64);
      cs = float(cs64);
    } else {
      sincosf(pos * inv_freq[d], &sn, &cs);
    }
    T* h = row + size_t(head) * hd;
    const float a = to_float(h[d]), b = to_float(h[d + half]);
    const T ra = from_float<T>(a * cs - b * sn), rb = from_float<T>(b * cs + a * sn);
    h[d] = ra;
    h[d + half] = rb;
    if (head >= nq && slot >= 0) {
      T* dst = k_pool + ((size_t(page) * nkv + (head - nq)) * page_size + off) * hd;
      dst[d] = ra;
      dst[d + half] = rb;
    }
  }
  if (slot < 0) return;
  // the part of k heads beyond rotary_dim is cached as it is
  if (rotary_dim < hd) {
    const int rest = hd - rotary_dim;
    for (int i = threadIdx.x; i < nkv * rest; i += blockDim.x) {
      const int g = i / rest, d = rotary_dim + i % rest;
      k_pool[((size_t(page) * nkv + g) * page_size + off) * hd + d] = row[size_t(nq + g) * hd + d];
    }
  }
  for (int i = threadIdx.x; i < nkv * hd; i += blockDim.x) {
    const int g = i / hd, d = i % hd;
    v_pool[((size_t(page) * nkv + g) * hd + d) * page_size + off] = row[size_t(nq + nkv + g) * hd + d];
  }
}

}  // namespace sprout

namespace sprout {
// tokens[i] = previous[source[i]] where source[i] >= 0 (a token that an earlier step sampled and the host
// has not read yet); an invalid token (the sampler's mark for non-finite logits) becomes 0: the step's
// result is thrown away by the host, but its kernels must not index with it.
__global__ void feed_tokens_kernel(int32_t* __restrict__ tokens, const int32_t* __restrict__ previous,
                                   const int32_t* __restrict__ source, int n, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int from = source[i];
  if (from < 0) return;
  const int token = previous[from];
  tokens[i] = token >= 0 && token < vocab ? token : 0;
}
}  // namespace sprout

using namespace sprout;

extern "C" int sp_feed_tokens(void* stream, int32_t* tokens, const int32_t* previous, const int32_t* source, int n,
                              int vocab) {
  SP_REQUIRE(n >= 0 && vocab > 0 && tokens && previous && source, "sp_feed_tokens: bad arguments");
  if (n == 0) return 0;
  feed_tokens_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(tokens, previous, source, n, vocab);
  return check_launch("sp_feed_tokens");
}

extern "C" int sp_embed(void* stream, int table_dtype, const void* table, const int32_t* tokens,
                        float* residual, int T, int H, int V) {
  SP_REQUIRE(T >= 0 && H > 0 && V > 0, "sp_embed: bad sizes T=%d H=%d V=%d", T, H, V);
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == kF32)
    embed_kernel<float><<<T, 256, 0, s>>>((const float*)table, tokens, residual, H);
  else if (table_dtype == kBF16)
    embed_kernel<bf16_t><<<T, 256, 0, s>>>((const bf16_t*)table, tokens, residual, H);
  else
    SP_REQUIRE(false, "sp_embed: unsupported table dtype %d", table_dtype);
  return check_launch("sp_embed");
}

extern "C" int sp_rmsnorm(void* stream, const float* x, const int32_t* rows, int w_dtype, const void* w,
                          float eps, int out_dtype, void* out, int R, int H) {
  SP_REQUIRE(R >= 0 && H > 0, "sp_rmsnorm: bad sizes R=%d H=%d", R, H);
  if (R == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  const int threads = H >= 1024 ? 512 : 256;
  // rows of whole groups of four that the threads of a block hold in registers: one trip to memory
  const int per = H % 4 == 0 ? (H / 4 + threads - 1) / threads : 0;
#define SP_NORM(TW, TO)                                                                                          \
  do {                                                                                                           \
    if (per == 1) rmsnorm_rows_kernel<TW, TO, 1><<<R, threads, 0, s>>>(x, rows, (const TW*)w, eps, (TO*)out, H);  \
    else if (per == 2) rmsnorm_rows_kernel<TW, TO, 2><<<R, threads, 0, s>>>(x, rows, (const TW*)w, eps, (TO*)out, H); \
    else if (per >= 3 && per <= 4) rmsnorm_rows_kernel<TW, TO, 4><<<R, threads, 0, s>>>(x, rows, (const TW*)w, eps, (TO*)out, H); \
    else rmsnorm_kernel<TW, TO><<<R, threads, 0, s>>>(x, rows, (const TW*)w, eps, (TO*)out, H);                   \
  } while (0)
  if (w_dtype == kF32 && out_dtype == kF32) SP_NORM(float, float);
  else if (w_dtype == kF32 && out_dtype == kBF16) SP_NORM(float, bf16_t);
  else if (w_dtype == kBF16 && out_dtype == kF32) SP_NORM(bf16_t, float);
  else if (w_dtype == kBF16 && out_dtype == kBF16) SP_NORM(bf16_t, bf16_t);
  else SP_REQUIRE(false, "sp_rmsnorm: unsupported dtypes w=%d out=%d", w_dtype, out_dtype);
#undef SP_NORM
  return check_launch("sp_rmsnorm");
}

extern "C" int sp_silu_mul(void* stream, int dtype, const void* gu, void* out, int T, int I, int activation) {
  SP_REQUIRE(activation == 0, "sp_silu_mul: no kernel for activation %d (0 = SiLU)", activation);
  SP_REQUIRE(T >= 0 && I > 0, "sp_silu_mul: bad sizes T=%d I=%d", T, I);
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((I + 255) / 256, T);
  if (dtype == kF32) silu_mul_kernel<float><<<grid, 256, 0, s>>>((const float*)gu, (float*)out, I);
  else if (dtype == kBF16) silu_mul_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)gu, (bf16_t*)out, I);
  else SP_REQUIRE(false, "sp_silu_mul: unsupported dtype %d", dtype);
  return check_launch("sp_silu_mul");
}

extern "C" int sp_rope_table(void* stream, const int32_t* positions, const float* inv_freq, int half, float* out, int T) {
  SP_REQUIRE(T >= 0 && half > 0 && positions && inv_freq && out, "sp_rope_table: bad arguments");
  SP_REQUIRE(int64_t(T) * half < (int64_t(1) << 31), "sp_rope_table: too many entries");
  if (T == 0) return 0;
  const int n = T * half;
  rope_table_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(positions, inv_freq, half, reinterpret_cast<float2*>(out), n);
  return check_launch("sp_rope_table");
}

extern "C" int sp_rope_cache(void* stream, int dtype, void* qkv, const int32_t* positions,
                             const float* inv_freq, const float* inv_freq_tail, int rotary_dim,
                             const int32_t* slot_mapping, void* k_pool,
                             void* v_pool, int T, int nq, int nkv, int hd, int page_size, int num_pages, int pairing) {
  SP_REQUIRE(pairing == 0, "sp_rope_cache: no kernel for pairing %d (0 = halves of the rotated dimensions)", pairing);
  SP_REQUIRE(T >= 0 && nq > 0 && nkv >= 0 && hd > 0, "sp_rope_cache: bad sizes");
  SP_REQUIRE(rotary_dim >= 0 && rotary_dim <= hd && rotary_dim % 2 == 0,
             "sp_rope_cache: rotary_dim %d must be even and at most head size %d", rotary_dim, hd);
  SP_REQUIRE(nkv == 0 || (slot_mapping && k_pool && v_pool && page_size > 0 && num_pages > 0),
             "sp_rope_cache: cache arguments missing");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == kF32)
    rope_cache_kernel<float><<<T, 256, 0, s>>>((float*)qkv, positions, inv_freq, inv_freq_tail, rotary_dim, slot_mapping,
                                               (float*)k_pool, (float*)v_pool, nq, nkv, hd, page_size);
  else if (dtype == kBF16 && hd % 8 == 0 && rotary_dim % 8 == 0 && rotary_dim <= 1024)   // at most 128 groups of four pairs
    rope_cache_bf16_kernel<<<T, 128, 0, s>>>((bf16_t*)qkv, positions, inv_freq, rotary_dim, slot_mapping, (bf16_t*)k_pool,
                                             (bf16_t*)v_pool, nq, nkv, hd, page_size);
  else if (dtype == kBF16)
    rope_cache_kernel<bf16_t><<<T, 256, 0, s>>>((bf16_t*)qkv, positions, inv_freq, nullptr, rotary_dim, slot_mapping,
                                                (bf16_t*)k_pool, (bf16_t*)v_pool, nq, nkv, hd, page_size);
  else
    SP_REQUIRE(false, "sp_rope_cache: unsupported dtype %d", dtype);
  return check_launch("sp_rope_cache");
}
