// Matrix-core (MFMA) operand types and the bf16 instructions of gfx950.
#pragma once

#include "common.h"

namespace bc4g {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

// D[16x16] += A[16x32] * B[32x16], bf16 in, float accumulate.  Lane l holds, of A, row l%16 and
// the eight k-slots of group l/16; of B, column l%16 and the same eight k-slots; of D, column
// l%16 and rows 4*(l/16) + 0..3.  Which k a slot stands for is the caller's choice, as long as A
// and B agree.
__device__ inline floatx4 mfma_16x16x32(uint4 a, uint4 b, floatx4 acc) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                 acc, 0, 0, 0);
}

// D[32x32] += A[32x16] * B[16x32].  Lane l holds, of A, row l%32 and the eight k-slots of group
// l/32; of B, column l%32 and the same slots; of D, column l%32 and rows 8*(r/4) + 4*(l/32) + r%4
// for r = 0..15.
__device__ inline floatx16 mfma_32x32x16(uint4 a, uint4 b, floatx16 acc) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                 acc, 0, 0, 0);
}

__device__ inline uint4 load16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline uint4 zero16() { return make_uint4(0u, 0u, 0u, 0u); }

}  // namespace bc4g
