// Matrix-core (MFMA) helpers for gfx950: operand vector types and 16-byte loads.
#pragma once
#include "common.h"

namespace sprout {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// v_mfma_f32_16x16x32_bf16: D[16x16] += A[16x32] . B[32x16].
// Lane l holds A[l % 16][8 * (l / 16) .. + 8] and B[8 * (l / 16) .. + 8][l % 16];
// D lane l, element r: row 4 * (l / 16) + r, column l % 16.
__device__ __forceinline__ floatx4 mfma16(bf16x8 a, bf16x8 b, floatx4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
// v_mfma_f32_32x32x16_bf16: D[32x32] += A[32x16] . B[16x32].
// Lane l holds A[l % 32][8 * (l / 32) .. + 8] and B[8 * (l / 32) .. + 8][l % 32];
// D lane l, element r: row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32.
__device__ __forceinline__ floatx16 mfma32(bf16x8 a, bf16x8 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// v_mfma_f32_32x32x2_f32: D[32x32] += A[32x2] . B[2x32] with float32 operands (a true 32-bit product).
// Lane l holds A[l % 32][l / 32] and B[l / 32][l % 32]; D as above.
__device__ __forceinline__ floatx16 mfma32_f32(float a, float b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ __forceinline__ uint4 ldg128(const void* p) { return *reinterpret_cast<const uint4*>(p); }

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
// Two floats to two bfloat16 (round to nearest even) in one instruction.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

}  // namespace sprout
