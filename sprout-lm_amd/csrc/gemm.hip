// Entry point of the matrix products: checks the operands and picks a kernel.
#include "common.h"
#include "sprout_hip.h"

namespace sprout {
int gemm_generic(hipStream_t s, int a_dtype, const void* a, int w_dtype, const void* w, int bias_dtype,
                 const void* bias, int mode, int out_dtype, void* out, int T, int N, int K);
int gemm_bf16(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode,
              int out_dtype, void* out, int T, int N, int K, bool* handled);
bool gemm_f32_takes(int T, int N, int K, const void* a, const void* w, const void* out);
bool gemm_f32_skinny_takes(int T, int N, int K, const void* a, const void* w);
int gemm_f32_skinny(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out,
                    int T, int N, int K);
int gemm_f32(hipStream_t s, const void* a, const void* w, int bias_dtype, const void* bias, int mode, void* out, int T,
             int N, int K);
}  // namespace sprout

using namespace sprout;

extern "C" int sp_gemm(void* stream, int a_dtype, const void* a, int w_dtype, const void* w, int bias_dtype,
                       const void* bias, int mode, int out_dtype, void* out, int T, int N, int K) {
  SP_REQUIRE(T >= 0 && N > 0 && K > 0, "sp_gemm: bad sizes T=%d N=%d K=%d", T, N, K);
  SP_REQUIRE((a_dtype == kF32 || a_dtype == kBF16) && (w_dtype == kF32 || w_dtype == kBF16),
             "sp_gemm: unsupported operand dtypes a=%d w=%d", a_dtype, w_dtype);
  SP_REQUIRE(mode >= 0 && mode <= 2, "sp_gemm: unknown mode %d", mode);
  SP_REQUIRE(mode != 0 || out_dtype == kF32 || out_dtype == kBF16, "sp_gemm: unsupported output dtype %d", out_dtype);
  SP_REQUIRE(!bias || bias_dtype == kF32 || bias_dtype == kBF16, "sp_gemm: unsupported bias dtype %d", bias_dtype);
  SP_REQUIRE(a && w && out, "sp_gemm: null operand");
  if (T == 0) return 0;
  hipStream_t s = (hipStream_t)stream;
  if (a_dtype == kBF16 && w_dtype == kBF16) {
    bool handled = false;
    int rc = gemm_bf16(s, a, w, bias_dtype, bias, mode, out_dtype, out, T, N, K, &handled);
    if (handled) return rc;
  }
  // float32 operands and a float32 result, more than a handful of tokens: the matrix cores' true 32-bit products
  if (a_dtype == kF32 && w_dtype == kF32 && (mode != 0 || out_dtype == kF32)) {
    if (gemm_f32_skinny_takes(T, N, K, a, w)) return gemm_f32_skinny(s, a, w, bias_dtype, bias, mode, out, T, N, K);
    if (gemm_f32_takes(T, N, K, a, w, out)) return gemm_f32(s, a, w, bias_dtype, bias, mode, out, T, N, K);
  }
  return gemm_generic(s, a_dtype, a, w_dtype, w, bias_dtype, bias, mode, out_dtype, out, T, N, K);
}
