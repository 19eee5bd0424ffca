// The plain modes of the pipelined tiled product with a bfloat16 bias (the kernel of gemm_pipe.h, the shapes
// of gemm_pipe.hip): a file of its own, so that it compiles beside the others.
#include "gemm_pipe.h"

namespace sprout {

int gemm_bf16_pipe_bias16(hipStream_t s, const void* a, const void* w, const void* bias, int mode, void* out, int T, int N,
                          int K) {
  return pipe_shape<bf16_t>(s, a, w, bias, mode, out, T, N, K);
}

}  // namespace sprout
