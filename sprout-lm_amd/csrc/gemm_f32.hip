// Tiled float32 product for more than a handful of tokens: out[T, N] (float32) = or += x[T, K] . w[N, K]^T with
// float32 operands, on v_mfma_f32_32x32x2_f32 (true 32-bit products and sums; no reduced-precision mode).  The
// kernel is the pipelined tiled product of gemm_pipe.h with float operands; K must be a multiple of 32 (rows of
// whole 128-byte slices).  Everything else (few tokens, other K, mixed operand types) stays on the FMA kernels.
#include "gemm_pipe.h"

namespace sprout {

namespace {

struct F32Shape { int bm, bn; float cost; };   // cost: time of a block per unit of area, against the largest shape
constexpr F32Shape kShapes[4] = {{256, 128, 1.0f}, {128, 128, 1.05f}, {64, 128, 1.12f}, {64, 64, 1.25f}};

// The matrix cores bound this product, so a launch takes as long as the CU with the most tile area: the shape
// with the least (blocks on the fullest CU) x (tile area) x (what a smaller tile loses to its fetches).
int choose_shape(int T, int N) {
  int best = 0;
  float best_cost = 0.f;
  for (int i = 0; i < 4; ++i) {
    const long blocks = long((T + kShapes[i].bm - 1) / kShapes[i].bm) * ((N + kShapes[i].bn - 1) / kShapes[i].bn);
    const float cost = float((blocks + 255) / 256) * kShapes[i].bm * kShapes[i].bn * kShapes[i].cost;
    if (i == 0 || cost < best_cost) { best = i; best_cost = cost; }
  }
  return best;
}

template <int WM, int WN, int WAVES_M, int WAVES_N, int STAGES, typename TB>
int launch_f32(hipStream_t s, const float* x, const float* w, const void* bias, int mode, float* out, int T, int N, int K) {
  if (mode == kAccumulate)
    return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kAccumulate, TB, float>(s, 1, x, w, (const TB*)bias, out, T, N, K, K);
  return launch_pipe_mode<WM, WN, WAVES_M, WAVES_N, STAGES, kStoreF32, TB, float>(s, 1, x, w, (const TB*)bias, out, T, N, K, K);
}

template <typename TB>
int launch_shape(hipStream_t s, const float* x, const float* w, const void* bias, int mode, float* out, int T, int N, int K) {
  switch (choose_shape(T, N)) {
    case 0: return launch_f32<2, 2, 4, 2, 3, TB>(s, x, w, bias, mode, out, T, N, K);
    case 1: return launch_f32<1, 2, 4, 2, 4, TB>(s, x, w, bias, mode, out, T, N, K);
    case 2: return launch_f32<1, 2, 2, 2, 3, TB>(s, x, w, bias, mode, out, T, N, K);
    default: return launch_f32<1, 1, 2, 2, 4, TB>(s, x, w, bias, mode, out, T, N, K);
  }
}

}  // namespace

bool gemm_f32_takes(int T, int N, int K, const void* a, const void* w, const void* out) {
  return T > 16 && K % 32 == 0 && K >= 32 && int64_t(K) * 4 * 256 < (int64_t(1) << 32) &&
         (reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
}

// mode: kAccumulate (out += ...) or anything else (out = ...); out is float32 either way.
int gemm_f32(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out, int T,
             int N, int K) {
  if (bias && bias_dtype == kBF16)
    return launch_shape<bf16_t>(s, (const float*)a, (const float*)w, bias, mode, (float*)out, T, N, K);
  return launch_shape<float>(s, (const float*)a, (const float*)w, bias, mode, (float*)out, T, N, K);
}

}  // namespace sprout
