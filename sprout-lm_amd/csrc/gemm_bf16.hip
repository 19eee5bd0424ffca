// bfloat16 matrix products on the matrix cores: out[T, N] = x[T, K] . w[N, K]^T, float32 sums.
//
// "Skinny" kernel (T <= 64, decoding): the step is bound by reading w once, so every wave streams
// its rows of w straight from memory into registers (16-byte loads, a 128-byte line per row and
// instruction), the few activations wait in LDS, and the product runs on 16x16x32 MFMA with the
// weights as the A operand: D[n, t].  Small matrices are cut along K over several blocks, whose
// partial sums are added into the float32 output with hardware atomics (accumulate mode only).
#include "gemm_epilogue.h"
#include "sprout_hip.h"

namespace sprout {


template <int TN> struct SkinnyChunk { static constexpr int KC = TN >= 3 ? 448 : 512; };

// grid: (blocks of 4 * RW row tiles, K splits).  block: 256 threads = 4 waves, each RW tiles of 16 rows.
template <int TN, int RW, int MODE, typename TB>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const uint16_t* __restrict__ x,
                                                          const uint16_t* __restrict__ w,
                                                          const TB* __restrict__ bias, void* __restrict__ out,
                                                          int T, int N, int K, int k_per_split) {
  constexpr int KC = SkinnyChunk<TN>::KC;
  constexpr int LD = KC / 8 + 1;                      // row pitch of the staged activations, in uint4
  extern __shared__ uint4 xs[];                       // [TN * 16][LD]
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int lr = lane & 15, lj = lane >> 4;
  const int tile0 = (blockIdx.x * 4 + wave) * RW;
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);

  const uint16_t* wrow[RW];
#pragma unroll
  for (int rw = 0; rw < RW; ++rw) wrow[rw] = w + size_t(min(N - 1, (tile0 + rw) * 16 + lr)) * K;

  floatx4 acc[RW][TN];
#pragma unroll
  for (int rw = 0; rw < RW; ++rw)
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) acc[rw][tn] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int kc = k_begin; kc < k_end; kc += KC) {
    __syncthreads();
    for (int i = threadIdx.x; i < TN * 16 * (KC / 8); i += 256) {
      const int t = i / (KC / 8), c = i % (KC / 8), k = kc + c * 8;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (t < T && k < k_end) v = ldg128(x + size_t(t) * K + k);   // K and the split are multiples of 8
      xs[t * LD + c] = v;
    }
    __syncthreads();
    const int klen = min(KC, k_end - kc);
    for (int kk = 0; kk < klen; kk += 64) {
      const int k = kc + kk + 16 * lj;                // this lane's 16 elements of the 64-wide step
      const bool in0 = k < k_end, in1 = k + 8 < k_end;
      uint4 a0[RW], a1[RW];
#pragma unroll
      for (int rw = 0; rw < RW; ++rw) {
        a0[rw] = in0 ? ldg128(wrow[rw] + k) : make_uint4(0, 0, 0, 0);
        a1[rw] = in1 ? ldg128(wrow[rw] + k + 8) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) {
        const uint4 b0 = xs[(tn * 16 + lr) * LD + (kk >> 3) + 2 * lj];
        const uint4 b1 = xs[(tn * 16 + lr) * LD + (kk >> 3) + 2 * lj + 1];
#pragma unroll
        for (int rw = 0; rw < RW; ++rw) {
          acc[rw][tn] = mfma16(as_bf16x8(a0[rw]), as_bf16x8(b0), acc[rw][tn]);
          acc[rw][tn] = mfma16(as_bf16x8(a1[rw]), as_bf16x8(b1), acc[rw][tn]);
        }
      }
    }
  }

  // lane holds out[t = tn * 16 + lr][n = tile * 16 + 4 * lj + r], r = 0..3
#pragma unroll
  for (int rw = 0; rw < RW; ++rw) {
    const int n0 = (tile0 + rw) * 16 + 4 * lj;
    if (n0 >= N) continue;
#pragma unroll
    for (int tn = 0; tn < TN; ++tn) {
      const int t = tn * 16 + lr;
      if (t >= T) continue;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] = acc[rw][tn][r];
        if (bias && blockIdx.y == 0 && n0 + r < N) v[r] += to_float(bias[n0 + r]);
      }
      const size_t o = size_t(t) * N + n0;
      if (MODE == kStore) {
        uint16_t* dst = reinterpret_cast<uint16_t*>(out) + o;
        if (n0 + 4 <= N && (N & 3) == 0) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        } else {
          for (int r = 0; r < 4 && n0 + r < N; ++r) dst[r] = f32_to_bf16_bits(v[r]);
        }
      } else if (MODE == kStoreF32) {
        float* dst = reinterpret_cast<float*>(out) + o;
        if (n0 + 4 <= N && (N & 3) == 0) {
          *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
          for (int r = 0; r < 4 && n0 + r < N; ++r) dst[r] = v[r];
        }
      } else {
        float* dst = reinterpret_cast<float*>(out) + o;
        if (gridDim.y == 1) {
          for (int r = 0; r < 4 && n0 + r < N; ++r) dst[r] += v[r];
        } else {
          for (int r = 0; r < 4 && n0 + r < N; ++r) unsafeAtomicAdd(dst + r, v[r]);
        }
      }
    }
  }
}

template <int TN, int RW, int MODE, typename TB>
static int launch_skinny(hipStream_t s, const void* x, const void* w, const void* bias, void* out, int T, int N, int K,
                         int splits, int k_per_split) {
  constexpr int KC = SkinnyChunk<TN>::KC;
  const int tiles = (N + 15) / 16;
  dim3 grid((tiles + 4 * RW - 1) / (4 * RW), splits);
  const size_t lds = size_t(TN) * 16 * (KC / 8 + 1) * sizeof(uint4);
  gemm_skinny_kernel<TN, RW, MODE, TB><<<grid, 256, lds, s>>>((const uint16_t*)x, (const uint16_t*)w, (const TB*)bias,
                                                               out, T, N, K, k_per_split);
  return check_launch("sp_gemm (skinny)");
}

template <int TN, int RW, typename TB>
static int skinny_mode(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T, int N,
                       int K, int splits, int k_per_split) {
  if (mode == kStore) return launch_skinny<TN, RW, kStore, TB>(s, x, w, bias, out, T, N, K, splits, k_per_split);
  if (mode == kAccumulate) return launch_skinny<TN, RW, kAccumulate, TB>(s, x, w, bias, out, T, N, K, splits, k_per_split);
  return launch_skinny<TN, RW, kStoreF32, TB>(s, x, w, bias, out, T, N, K, splits, k_per_split);
}

template <typename TB>
static int skinny_shape(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T, int N,
                        int K) {
  const int tiles = (N + 15) / 16;
  const int rw = tiles >= 4096 ? 2 : 1;
  int splits = 1, k_per_split = K;
  if (mode == kAccumulate) {
    const int want = (1536 + tiles - 1) / tiles;          // enough waves to keep every SIMD loading
    splits = max(1, min(want, K / 256));
    k_per_split = ((K + splits - 1) / splits + 63) / 64 * 64;
    splits = (K + k_per_split - 1) / k_per_split;
  }
#define SP_SKINNY(TN)                                                                                              \
  (rw == 2 ? skinny_mode<TN, 2, TB>(s, x, w, bias, mode, out, T, N, K, splits, k_per_split)                        \
           : skinny_mode<TN, 1, TB>(s, x, w, bias, mode, out, T, N, K, splits, k_per_split))
  if (T <= 16) return SP_SKINNY(1);
  if (T <= 32) return SP_SKINNY(2);
  return SP_SKINNY(4);
#undef SP_SKINNY
}

int gemm_bf16_tiled(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                    int T, int N, int K);
int gemm_decode_plain(hipStream_t s, const void* x, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                      int T, int N, int K);
bool gemm_pipe_takes(int T, int N, int K);
int gemm_bf16_pipe(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                   int T, int N, int K);
int gemm_bf16_pipe_silu(hipStream_t s, const void* x, const void* w, void* out, int T, int I, int K);

// mode 0 stores bfloat16 here; a float32 store of mode 0 is passed in as mode 2 by the caller.
int gemm_bf16(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, int out_dtype,
              void* out, int T, int N, int K, bool* handled) {
  *handled = false;
  if (K % 8 != 0) return 0;                               // rows of w must start on 16-byte boundaries
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) & 15) return 0;
  if (mode == kStore && out_dtype == kF32) mode = kStoreF32;
  *handled = true;
  if (T <= 64) {
    // Few rows.  Large accumulating products stream their weights through the pipelined tiles (K split over
    // blocks), whatever the number of tokens (3,584 x 18,944: 25.4 against 27.7 us at one token, 26.0 against 29.7
    // at 8, 26.6 against 32.8 at 16); the others split K between the waves of a block.
    // (up to 16 tokens only where the matrix is that large: 3,584 x 3,584 at 8 tokens is 8.2 us fused, 8.8 tiled)
    if (mode == kAccumulate && size_t(N) * K >= (size_t(T > 16 ? 6 : 32) << 20) && gemm_pipe_takes(T, N, K))
      return gemm_bf16_pipe(s, a, w, bias_dtype, bias, mode, out, T, N, K);
    if ((N + 15) / 16 < 2048) return gemm_decode_plain(s, a, w, bias_dtype, bias, mode, out, T, N, K);
    // Very wide (the output head): rows streamed per wave up to 16 tokens; with more, the streaming kernel stops
    // for every chunk of activations it stages, and the pipelined tiles are faster (151,936 x 896 at 64 tokens:
    // 98 against 126 us, 152,064 x 3,584: 263 against 409; the same at 16 tokens and fewer).
    if (T > 16 && gemm_pipe_takes(T, N, K)) return gemm_bf16_pipe(s, a, w, bias_dtype, bias, mode, out, T, N, K);
    if (bias && bias_dtype == kBF16) return skinny_shape<bf16_t>(s, a, w, bias, mode, out, T, N, K);
    return skinny_shape<float>(s, a, w, bias, mode, out, T, N, K);
  }
  if (gemm_pipe_takes(T, N, K)) return gemm_bf16_pipe(s, a, w, bias_dtype, bias, mode, out, T, N, K);
  return gemm_bf16_tiled(s, a, w, bias_dtype, bias, mode, out, T, N, K);
}

}  // namespace sprout

// ------------------------------------------------------------------------------------------------
// Tiled kernel for the shapes that the pipelined kernel (gemm_pipe.hip) does not take: T > 64 with a K that is
// no multiple of 64.  Both operands go through LDS in steps of 64 or 128 along K; 4 waves in a
// 2 x 2 arrangement, each computing WM x WN tiles of 32 x 32 on 32x32x16 MFMA with the weights as the
// A operand (D[n, t]), so that a lane ends with four consecutive n of one token and stores 8 or 16 bytes.
// The next step is on its way from memory while one is multiplied.  Small accumulating products may be
// split along K over blockIdx.z (hardware float atomics).
namespace sprout {


template <int WM, int WN, int TBK, int MODE, typename TB>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const uint16_t* __restrict__ x,
                                                         const uint16_t* __restrict__ w,
                                                         const TB* __restrict__ bias, void* __restrict__ out, int T,
                                                         int N, int K, int k_per_split) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int TPITCH = TBK + 8;    // LDS row pitch in elements: rows stay 16-byte aligned, banks shift by 4
  constexpr int CPR = TBK / 8;       // 16-byte pieces per row of a step
  constexpr int XL = BM * CPR / 256, WL = BN * CPR / 256;   // 16-byte loads per thread and operand
  // two buffers of (activation tile, weight tile): one is multiplied while the other is filled
  extern __shared__ __attribute__((aligned(16))) uint16_t tiles_lds[];
  constexpr int BUF = (BM + BN) * TPITCH;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int li = lane & 31, lk = lane >> 5;
  const int t0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int k_begin = blockIdx.z * k_per_split, k_end = min(K, k_begin + k_per_split);

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // what this thread copies: rows tid / CPR + (256 / CPR) i of each operand tile, columns 8 (tid % CPR) .. + 7
  constexpr int RSTEP = 256 / CPR;
  const int crow = threadIdx.x / CPR, ccol = (threadIdx.x % CPR) * 8;
  const uint16_t* xsrc[XL];
  const uint16_t* wsrc[WL];
#pragma unroll
  for (int i = 0; i < XL; ++i) xsrc[i] = t0 + crow + RSTEP * i < T ? x + size_t(t0 + crow + RSTEP * i) * K + ccol : nullptr;
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int r = crow + RSTEP * i;          // row of the weight tile in LDS
    int row = n0 + r;                        // its row in w
    bool in = row < N;
    if (MODE == kSilu) {
      // N counts gate rows; w holds N gate rows, then N up rows.  Tile rows alternate in runs of 32
      // between gate rows and the matching up rows, so that a lane ends with both of one index.
      const int gate = blockIdx.x * (BN / 2) + (r / 64) * 32 + (r & 31);
      in = gate < N;
      row = ((r >> 5) & 1) ? N + gate : gate;
    }
    wsrc[i] = in ? w + size_t(row) * K + ccol : nullptr;
  }

  struct Regs { uint4 x[XL]; uint4 w[WL]; };
  auto load_global = [&](Regs& r, int k0) {
    const bool kin = k0 + ccol < k_end;
#pragma unroll
    for (int i = 0; i < XL; ++i) r.x[i] = (xsrc[i] && kin) ? ldg128(xsrc[i] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < WL; ++i) r.w[i] = (wsrc[i] && kin) ? ldg128(wsrc[i] + k0) : make_uint4(0, 0, 0, 0);
  };
  auto store_lds = [&](const Regs& r, int buf) {
    uint16_t* xs = tiles_lds + buf * BUF;
    uint16_t* ws = xs + BM * TPITCH;
#pragma unroll
    for (int i = 0; i < XL; ++i) *reinterpret_cast<uint4*>(xs + (crow + RSTEP * i) * TPITCH + ccol) = r.x[i];
#pragma unroll
    for (int i = 0; i < WL; ++i) *reinterpret_cast<uint4*>(ws + (crow + RSTEP * i) * TPITCH + ccol) = r.w[i];
  };
  auto multiply = [&](int buf) {
    const uint16_t* xs = tiles_lds + buf * BUF;
    const uint16_t* ws = xs + BM * TPITCH;
#pragma unroll
    for (int ks = 0; ks < TBK / 16; ++ks) {
      bf16x8 a[WM], b[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[i] = as_bf16x8(*reinterpret_cast<const uint4*>(xs + ((wm * WM + i) * 32 + li) * TPITCH + ks * 16 + lk * 8));
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[j] = as_bf16x8(*reinterpret_cast<const uint4*>(ws + ((wn * WN + j) * 32 + li) * TPITCH + ks * 16 + lk * 8));
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = mfma32(b[j], a[i], acc[i][j]);
    }
  };

  // The next step's loads are in flight while the current one is multiplied, and go into the other
  // LDS buffer afterwards: one barrier per step.  (A second set of staging registers, to have two
  // steps in flight, cost more in occupancy than it hid: 93 us against 74 us on 2048 x 9728 x 896.)
  Regs r;
  load_global(r, k_begin);
  store_lds(r, 0);
  __syncthreads();
  int buf = 0;
  for (int k0 = k_begin; k0 < k_end; k0 += TBK, buf ^= 1) {
    const bool more = k0 + TBK < k_end;
    if (more) load_global(r, k0 + TBK);
    multiply(buf);
    if (more) store_lds(r, buf ^ 1);
    __syncthreads();
  }

  static_assert(4 * 32 * (32 * WN + 4) * sizeof(float) <= 2 * BUF * sizeof(uint16_t), "the turning buffer must fit");
  tile_epilogue<WM, WN, MODE, TB>(acc, reinterpret_cast<float*>(tiles_lds), bias, out, T, N, t0, n0);
}

template <int WM, int WN, int TBK, int MODE, typename TB>
static int launch_tiled_mode(hipStream_t s, dim3 grid, const uint16_t* x, const uint16_t* w, const TB* bias, void* out,
                             int T, int N, int K, int k_per_split) {
  constexpr size_t lds = size_t(2) * 64 * (WM + WN) * (TBK + 8) * sizeof(uint16_t);
  static bool raised = false;
  if (lds > 48 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_tiled_kernel<WM, WN, TBK, MODE, TB>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (e != hipSuccess) {
      set_error("sp_gemm (tiled): cannot raise the LDS limit: %s", hipGetErrorString(e));
      return 1;
    }
    raised = true;
  }
  gemm_tiled_kernel<WM, WN, TBK, MODE, TB><<<grid, 256, lds, s>>>(x, w, bias, out, T, N, K, k_per_split);
  return check_launch("sp_gemm (tiled)");
}

template <int WM, int WN, int TBK, typename TB>
static int launch_tiled_bk(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T,
                           int N, int K, int splits) {
  const int k_per_split = ((K + splits - 1) / splits + TBK - 1) / TBK * TBK;
  splits = (K + k_per_split - 1) / k_per_split;
  dim3 grid((N + 64 * WN - 1) / (64 * WN), (T + 64 * WM - 1) / (64 * WM), splits);
  const uint16_t *xp = (const uint16_t*)x, *wp = (const uint16_t*)w;
  const TB* bp = (const TB*)bias;
  if (mode == kStore) return launch_tiled_mode<WM, WN, TBK, kStore, TB>(s, grid, xp, wp, bp, out, T, N, K, k_per_split);
  if (mode == kAccumulate) return launch_tiled_mode<WM, WN, TBK, kAccumulate, TB>(s, grid, xp, wp, bp, out, T, N, K, k_per_split);
  return launch_tiled_mode<WM, WN, TBK, kStoreF32, TB>(s, grid, xp, wp, bp, out, T, N, K, k_per_split);
}

// Long K: steps of 128 halve the number of barriers; only the small tiles have the LDS for it.
template <int WM, int WN, typename TB>
static int launch_tiled(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T, int N,
                        int K, int splits) {
  if (WM * WN <= 2 && K / splits >= 2048) return launch_tiled_bk<WM, WN, 128, TB>(s, x, w, bias, mode, out, T, N, K, splits);
  return launch_tiled_bk<WM, WN, 64, TB>(s, x, w, bias, mode, out, T, N, K, splits);
}

// Tile and split choice: large tiles reuse operands better, but the grid must fill 256 CUs several
// times over for loads to hide behind other blocks; accumulating products may also split K.
template <typename TB>
static int tiled_shape(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T, int N,
                       int K) {
  auto blocks = [&](int bm, int bn) { return ((T + bm - 1) / bm) * ((N + bn - 1) / bn); };
  // Splitting K pays only while the atomics stay few: T * N * splits float atomics cost more than
  // the product itself once T is in the thousands (measured 352 us against 44 us at 2048 x 896 x 4864).
  auto splits_for = [&](int nblocks) {
    if (mode != kAccumulate || size_t(T) * N > (size_t(1) << 20)) return 1;
    return max(1, min((768 + nblocks - 1) / nblocks, K / 512));
  };
  if (blocks(256, 128) >= 2048) return launch_tiled<4, 2, TB>(s, x, w, bias, mode, out, T, N, K, 1);
  if (blocks(128, 128) * splits_for(blocks(128, 128)) >= 384)
    return launch_tiled<2, 2, TB>(s, x, w, bias, mode, out, T, N, K, splits_for(blocks(128, 128)));
  if (blocks(128, 64) * splits_for(blocks(128, 64)) >= 256)
    return launch_tiled<2, 1, TB>(s, x, w, bias, mode, out, T, N, K, splits_for(blocks(128, 64)));
  return launch_tiled<1, 1, TB>(s, x, w, bias, mode, out, T, N, K, splits_for(blocks(64, 64)));
}

// out[T, I] = silu(x . w[:I]^T) * (x . w[I:]^T): the pipelined kernel where it takes the shape, else (T > 64)
// this file's kernel with 128-token tiles, 64 gate + 64 up rows per block.
int gemm_bf16_tiled_silu(hipStream_t s, const void* x, const void* w, void* out, int T, int I, int K) {
  if (gemm_pipe_takes(T, 2 * I, K)) return gemm_bf16_pipe_silu(s, x, w, out, T, I, K);
  dim3 grid((I + 63) / 64, (T + 127) / 128, 1);
  return launch_tiled_mode<2, 2, 64, kSilu, float>(s, grid, (const uint16_t*)x, (const uint16_t*)w, nullptr, out, T, I, K,
                                                    (K + 63) / 64 * 64);
}

int gemm_bf16_tiled(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                    int T, int N, int K) {
  if (bias && bias_dtype == kBF16) return tiled_shape<bf16_t>(s, a, w, bias, mode, out, T, N, K);
  return tiled_shape<float>(s, a, w, bias, mode, out, T, N, K);
}

}  // namespace sprout
