// Pipelined tiled bfloat16 product for many rows (prefill): out[T, N] = x[T, K] . w[N, K]^T with K a multiple of 64.
// The kernel and its launch; included by the files that instantiate its shapes.
//
// Memory latency, not arithmetic, bounds a tiled product whose blocks have only the next step in flight.  Here
// a block keeps STAGES - 1 steps of 64 along K in flight: tiles go from memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, so the depth costs LDS only), in a ring of STAGES buffers,
// and a step is multiplied while the next ones arrive.  One barrier per step.
//
// LDS layout of one stage: BM activation rows, then BN weight rows, each 128 bytes (64 elements) without
// padding.  One load instruction of a wave fills 1 KB = 8 rows: lane l writes bytes 16 l .. 16 l + 15, which
// is fixed by the hardware, so the layout is made conflict-free from the other side: lane l fetches, for row
// r = l / 8 of its group, the 16-byte piece (l % 8) ^ swz(r) of that row, i.e. piece p of row r lives at
// position p ^ swz(r).  swz(r) = (r ^ (r >> 3)) & 7 spreads the 16 rows that a quarter of a wave reads
// together over all banks, whether the LDS has 32 banks or 64.
//
// The compiler does not know of these loads (they are written in assembly: told of them, it would wait
// for all of them before every LDS read), so the kernel counts them itself: vmcnt before the barrier of a
// step allows exactly the loads of the later steps to be still on their way.
#pragma once
#include "gemm_epilogue.h"
#include "sprout_hip.h"

namespace sprout {

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// 64 lanes x 16 bytes from base + offset[lane] into LDS at lds_address + 16 lane.
__device__ __forceinline__ void load_to_lds(const void* base, uint32_t offset, uint32_t lds_address) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %0, %1"
      :
      : "v"(offset), "s"(base), "s"(lds_address)
      : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_loads_then_barrier() {
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(N) : "memory");
}

// How the tiles of a product are numbered over the blocks of a launch (the kernel and its launch agree on it):
// every XCD has `own` blocks for the weight tiles that are its own (`full` of them, token tiles in whole groups of
// `group`), then `run` blocks of the `left` weight tiles that are dealt out.
struct PipeTiles { int tiles_t, full, left, group, own, run; };
__host__ __device__ inline PipeTiles pipe_tiles(int tiles_t, int tiles_n) {
  PipeTiles p;
  p.tiles_t = tiles_t;
  p.full = tiles_n / 8;
  p.left = tiles_n % 8;
  p.group = tiles_t < 8 ? tiles_t : 8;
  p.own = p.full * p.group * ((tiles_t + p.group - 1) / p.group);
  p.run = (p.left * tiles_t + 7) / 8;
  return p;
}
// The tile of block `block` of the 8 (own + run) blocks of a launch, or false for a block with nothing to do.
__host__ __device__ inline bool pipe_tile_of(const PipeTiles& tiles, int block, int* tile_t, int* tile_n) {
  const int xcd = block & 7, i_xcd = block >> 3;
  if (i_xcd < tiles.own) {
    const int g = i_xcd / (tiles.full * tiles.group), rest = i_xcd % (tiles.full * tiles.group);
    *tile_n = (rest / tiles.group) * 8 + xcd;
    *tile_t = g * tiles.group + rest % tiles.group;
    return *tile_t < tiles.tiles_t;
  }
  const int j = i_xcd - tiles.own, k = xcd * tiles.run + j;
  if (j >= tiles.run || k >= tiles.left * tiles.tiles_t) return false;
  *tile_n = 8 * tiles.full + k / tiles.tiles_t;
  *tile_t = k % tiles.tiles_t;
  return true;
}

// A block of WAVES_M x WAVES_N waves, each with WM x WN tiles of 32 x 32: BM = 32 WM WAVES_M tokens by
// BN = 32 WN WAVES_N weight rows.  Blocks of up to four waves ask for the registers of two waves a SIMD: with
// all 512 to itself the compiler keeps the accumulators in one half of them and copies all of them to the
// other half and back around every turn of the ring.
//
// TE: the operands' element type.  uint16_t: bfloat16, steps of 64 along K on 32x32x16 MFMA.  float: the same
// bytes are steps of 32 along K, and a lane's 16-byte LDS read holds four numbers that feed four successive
// v_mfma_f32_32x32x2_f32 (k-slot l / 32 of MFMA e is element 4 (l / 32) + e of the eight that a 32-byte slice of a
// row holds, for both operands): true float32 products and sums, no reduced-precision mode, 1/8 of the bfloat16
// rate per byte, so this form is bound by the matrix cores and not by its fetches.
template <int WM, int WN, int WAVES_M, int WAVES_N, int STAGES, int MODE, typename TB, typename TE = uint16_t>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, (WAVES_M * WAVES_N <= 4 ? 2 : 1)) void gemm_pipe_kernel(const TE* __restrict__ x, const TE* __restrict__ w,
                                                        const TB* __restrict__ bias, void* __restrict__ out, int T,
                                                        int N, int K, int k_per_split, RopeArgs rope) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int ESZ = sizeof(TE), KSTEP = 128 / ESZ;    // elements of a tile row
  static_assert(ESZ == 2 || (MODE != kSilu && MODE != kRope && MODE != kStore), "float32 operands store or add float32");
  constexpr int BM = 32 * WM * WAVES_M, BN = 32 * WN * WAVES_N;
  constexpr int ROW = 128;                              // bytes of a tile row
  constexpr int STAGE = (BM + BN) * ROW;                // bytes of a stage
  constexpr int LX = BM / (8 * NW), LW = BN / (8 * NW); // load instructions per wave, stage and operand
  static_assert(BM % (8 * NW) == 0 && BN % (8 * NW) == 0, "every wave fills whole groups of 8 rows");
  static_assert((STAGES - 2) * (LX + LW) <= 63, "vmcnt holds six bits");
  extern __shared__ __attribute__((aligned(1024))) unsigned char pipe_lds[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int li = lane & 31, lk = lane >> 5;
  // Which tile: blocks go round the 8 XCDs (block b runs on XCD b % 8, each with an L2 of its own), so XCD c
  // takes the weight tiles c, c + 8, ... and nobody else fetches them; within an XCD the blocks that run
  // together are up to 8 token tiles of the same few weight tiles, so that w is read from memory once
  // whatever the number of tokens, and x stays in the caches.  The weight tiles left over when their number is no
  // multiple of 8 are dealt out by token tile, an equal run of their blocks to every XCD: four left-over weight
  // tiles would otherwise be a quarter more blocks on four of the XCDs, and fewer than 8 weight tiles idle XCDs.
  const PipeTiles tiles = pipe_tiles((T + BM - 1) / BM, ((MODE == kSilu ? 2 * N : N) + BN - 1) / BN);
  int tile_n, tile_t;
  if (!pipe_tile_of(tiles, blockIdx.x, &tile_t, &tile_n)) return;
  const int t0 = tile_t * BM, n0 = tile_n * BN;
  const int k_begin = blockIdx.z * k_per_split, k_end = min(K, k_begin + k_per_split);
  const int steps = (k_end - k_begin) / KSTEP;
  typedef __attribute__((address_space(3))) unsigned char* lds_address_t;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_address_t)pipe_lds;   // the tiles' offset within the LDS

  // ---- what this lane fetches: row 8 (NW j + wave) + lane / 8 of each operand tile, for j < LX (LW)
  const unsigned char* xbase = reinterpret_cast<const unsigned char*>(x + size_t(t0) * K + k_begin);
  const unsigned char* wbase = reinterpret_cast<const unsigned char*>(w + (MODE == kSilu || MODE == kRope ? size_t(0) : size_t(n0) * K) + k_begin);
  uint32_t xoff[LX], woff[LW];
#pragma unroll
  for (int j = 0; j < LX; ++j) {
    const int r = 8 * (NW * j + wave) + (lane >> 3);
    const int piece = (lane & 7) ^ swz(r);
    xoff[j] = uint32_t(min(r, T - 1 - t0)) * uint32_t(K) * uint32_t(ESZ) + piece * 16;
  }
#pragma unroll
  for (int j = 0; j < LW; ++j) {
    const int r = 8 * (NW * j + wave) + (lane >> 3);
    const int piece = (lane & 7) ^ swz(r);
    int row;
    if (MODE == kSilu) {
      // N counts gate rows; w holds N gate rows, then N up rows.  Tile rows alternate in runs of 32 between
      // gate rows and the matching up rows, so that a lane ends with both of one index.
      const int gate = min(N - 1, tile_n * (BN / 2) + (r / 64) * 32 + (r & 31));
      row = ((r >> 5) & 1) ? N + gate : gate;
    } else if (MODE == kRope) {
      // Tile rows in runs of 32: 32 dimensions of a head's first half, then their rotation partners half a
      // head further on, so that a lane ends with both of a pair.
      const int half = rope.hd / 2, groups_per_head = half / 32;
      const int group = tile_n * (BN / 64) + r / 64, head = group / groups_per_head, u = group % groups_per_head;
      row = min(N - 1, head * rope.hd + 32 * u + (r & 31) + ((r >> 5) & 1) * half);
    } else {
      row = min(r, N - 1 - n0);
    }
    woff[j] = uint32_t(row) * uint32_t(K) * uint32_t(ESZ) + piece * 16;
  }
  auto fetch = [&](int buf, int step) {
    const unsigned char* xs = xbase + size_t(step) * ROW;
    const unsigned char* ws = wbase + size_t(step) * ROW;
    const uint32_t dst = lds0 + buf * STAGE + wave * 8 * ROW;
#pragma unroll
    for (int j = 0; j < LX; ++j) load_to_lds(xs, xoff[j], dst + 8 * NW * j * ROW);
#pragma unroll
    for (int j = 0; j < LW; ++j) load_to_lds(ws, woff[j], dst + (BM + 8 * NW * j) * ROW);
  };

  // ---- what this lane reads for the MFMA operands: row 32 i + li of its wave's rows, pieces 2 ks + lk.
  // swz(32 m + li) = s0 ^ 4 (m & 1) with s0 = swz(li), so two positions per step serve all tiles of an operand,
  // and the tiles themselves are a constant number of bytes apart.
  const int s0 = swz(li);
  const uint32_t xrow0 = (wm * WM * 32 + li) * ROW, wrow0 = (BM + wn * WN * 32 + li) * ROW;
  const uint32_t xpos0 = ((lk ^ s0 ^ (4 * ((wm * WM) & 1))) << 4), wpos0 = ((lk ^ s0 ^ (4 * ((wn * WN) & 1))) << 4);

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  auto multiply = [&](int buf) {
    const unsigned char* stage = pipe_lds + buf * STAGE;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      uint4 a[WM], b[WN];
      const uint32_t xp = xrow0 + ((ks * 32) ^ xpos0), wp = wrow0 + ((ks * 32) ^ wpos0);
#pragma unroll
      for (int i = 0; i < WM; ++i)
        a[i] = *reinterpret_cast<const uint4*>(stage + ((i & 1) ? (xp ^ 64) : xp) + i * 32 * ROW);
#pragma unroll
      for (int j = 0; j < WN; ++j)
        b[j] = *reinterpret_cast<const uint4*>(stage + ((j & 1) ? (wp ^ 64) : wp) + j * 32 * ROW);
      if constexpr (ESZ == 2) {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j) acc[i][j] = mfma32(as_bf16x8(b[j]), as_bf16x8(a[i]), acc[i][j]);
      } else {
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
          for (int j = 0; j < WN; ++j) {
            acc[i][j] = mfma32_f32(__uint_as_float(b[j].x), __uint_as_float(a[i].x), acc[i][j]);
            acc[i][j] = mfma32_f32(__uint_as_float(b[j].y), __uint_as_float(a[i].y), acc[i][j]);
            acc[i][j] = mfma32_f32(__uint_as_float(b[j].z), __uint_as_float(a[i].z), acc[i][j]);
            acc[i][j] = mfma32_f32(__uint_as_float(b[j].w), __uint_as_float(a[i].w), acc[i][j]);
          }
      }
    }
  };

  // ---- the ring: step s lives in buffer s % STAGES; steps s + 1 .. s + STAGES - 2 are on their way while
  // step s is multiplied, and step s + STAGES - 1 is requested into the buffer that step s - 1 has left.
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < steps) fetch(s, s);
  for (int s0 = 0; s0 < steps; s0 += STAGES) {
#pragma unroll
    for (int u = 0; u < STAGES; ++u) {
      const int s = s0 + u;
      if (s >= steps) break;
      // every wave's loads of step s have landed, and every wave is done with step s - 1
      if (steps - 1 - s >= STAGES - 2) wait_loads_then_barrier<(STAGES - 2) * (LX + LW)>();
      else wait_loads_then_barrier<0>();
      if (s + STAGES - 1 < steps) fetch((u + STAGES - 1) % STAGES, s + STAGES - 1);
      multiply(u);
    }
  }
  if (MODE == kAccumulate && gridDim.z > 1) __syncthreads();   // the epilogue turns tiles round in this LDS
  static_assert(NW * 32 * (32 * WN + 4) * sizeof(float) <= size_t(STAGES) * STAGE, "the turning buffer must fit");
  tile_epilogue<WM, WN, MODE, TB, WAVES_N>(acc, reinterpret_cast<float*>(pipe_lds), bias, out, T, N, t0, n0, rope);
}

template <int WM, int WN, int WAVES_M, int WAVES_N, int STAGES, int MODE, typename TB, typename TE = uint16_t>
inline int launch_pipe_mode(hipStream_t s, int splits, const TE* x, const TE* w, const TB* bias, void* out,
                            int T, int N, int K, int k_per_split, const RopeArgs& rope = RopeArgs{}) {
  constexpr int BM = 32 * WM * WAVES_M, BN = 32 * WN * WAVES_N;
  constexpr size_t lds = size_t(STAGES) * (BM + BN) * 128;
  static bool raised = false;
  if (lds > 48 * 1024 && !raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_pipe_kernel<WM, WN, WAVES_M, WAVES_N, STAGES, MODE, TB, TE>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, int(lds));
    if (e != hipSuccess) {
      set_error("sp_gemm (pipelined): cannot raise the LDS limit: %s", hipGetErrorString(e));
      return 1;
    }
    raised = true;
  }
  // the kernel's own numbering of tiles
  const PipeTiles tiles = pipe_tiles((T + BM - 1) / BM, ((MODE == kSilu ? 2 * N : N) + BN - 1) / BN);
  dim3 grid(8 * (tiles.own + tiles.run), 1, splits);
  gemm_pipe_kernel<WM, WN, WAVES_M, WAVES_N, STAGES, MODE, TB, TE><<<grid, 64 * WAVES_M * WAVES_N, lds, s>>>(x, w, bias, out, T, N, K, k_per_split, rope);
  return check_launch("sp_gemm (pipelined)");
}


bool gemm_pipe_takes(int T, int N, int K);
// Picks the shape (index into the list in gemm_pipe.hip) and the split of K with the least estimated time.
// `paired`: the epilogue pairs tile columns, so shapes with one tile column a wave are left out.
void pipe_choice(int T, int N, int K, bool may_split, int* shape, int* splits, bool paired = false);

template <int WM, int WN, int WAVES_M, int WAVES_N, int STAGES, typename TB>
inline int launch_pipe(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T, int N,
                       int K, int splits) {
  const int k_per_split = ((K / 64 + splits - 1) / splits) * 64;
  splits = (K + k_per_split - 1) / k_per_split;
  const uint16_t *xp = (const uint16_t*)x, *wp = (const uint16_t*)w;
  const TB* bp = (const TB*)bias;
  if (mode == kStore) return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kStore, TB>(s, splits, xp, wp, bp, out, T, N, K, k_per_split);
  if (mode == kAccumulate) return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kAccumulate, TB>(s, splits, xp, wp, bp, out, T, N, K, k_per_split);
  return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kStoreF32, TB>(s, splits, xp, wp, bp, out, T, N, K, k_per_split);
}

template <typename TB>
inline int pipe_shape(hipStream_t s, const void* x, const void* w, const void* bias, int mode, void* out, int T, int N,
                      int K) {
  int shape, splits;
  pipe_choice(T, N, K, mode == kAccumulate, &shape, &splits);
  switch (shape) {
    case 0: return launch_pipe<4, 2, 2, 4, 2, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 1: return launch_pipe<2, 2, 4, 2, 3, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 2: return launch_pipe<1, 2, 4, 2, 4, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 4: return launch_pipe<1, 2, 2, 4, 3, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 5: return launch_pipe<1, 2, 2, 2, 3, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 6: return launch_pipe<6, 2, 2, 4, 2, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 7: return launch_pipe<1, 2, 2, 1, 4, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    case 8: return launch_pipe<2, 5, 4, 1, 3, TB>(s, x, w, bias, mode, out, T, N, K, splits);
    default: return launch_pipe<1, 1, 2, 2, 4, TB>(s, x, w, bias, mode, out, T, N, K, splits);
  }
}


}  // namespace sprout
