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

// x / (1 + e^-x) for the bfloat16 products' SwiGLU epilogues, by the hardware's 2^x and reciprocal (each good to a unit
// in the last place of a float; the result is rounded to bfloat16).  expf and a true division are an eighth of the
// tiled kernel's epilogue, and that a sixth of a wide gate-up product's time.
__device__ inline float silu_quick(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
}

__device__ inline uint4 load16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline uint4 zero16() { return make_uint4(0u, 0u, 0u, 0u); }

// Memory to LDS without passing registers: every lane of the wave brings the 16 bytes at its `global` to
// lds_address (the same in all lanes) + 16 * lane -- 1 KB of consecutive LDS a wave.
__device__ inline void load_to_lds_16(const void* global, unsigned lds_address) {
  // The LDS base of a wave-wide load travels in m0, which the compiler reserves for such uses of its
  // own and sets right before each (the kernels that call this give it none: no LDS load builtin, no
  // register array indexed at run time).  The compiler does not know the instruction, so the waits for it are written
  // by hand (wait_loads).
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(global), "s"(lds_address) : "memory");
}

// The same from one base address for the whole wave (in scalar registers) plus each lane's offset in bytes.
__device__ inline void load_to_lds_16(const void* wave_base, unsigned lane_offset, unsigned lds_address) {
  // (the base is the same in every lane; said so, half by half, it is kept in scalar registers)
  const uintptr_t bits = reinterpret_cast<uintptr_t>(wave_base);
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits >> 32));
  wave_base = reinterpret_cast<const void*>((static_cast<uintptr_t>(hi) << 32) | lo);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(wave_base), "s"(lds_address)
               : "memory");
}

// The same in two steps, for several loads to one stretch of LDS: the LDS address is set once, and each load adds
// OFFSET bytes (-4096 .. 4095) to it -- and to its memory address, so the caller takes OFFSET off that one.  (Setting
// the LDS address anew for every load costs the wave hundreds of clocks a load: the write to m0 waits for the load
// before it, which still needs the old value.)
__device__ inline void set_lds_base(unsigned lds_address) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" ::"s"(lds_address) : "memory");
}
template <int OFFSET>
__device__ inline void load_to_lds_16_at(const void* wave_base, unsigned lane_offset) {
  static_assert(OFFSET >= -4096 && OFFSET <= 4095, "the instruction's offset field");
  const uintptr_t bits = reinterpret_cast<uintptr_t>(wave_base) - OFFSET;
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits >> 32));
  wave_base = reinterpret_cast<const void*>((static_cast<uintptr_t>(hi) << 32) | lo);
  asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(lane_offset), "s"(wave_base), "n"(OFFSET) : "memory");
}

// Waits until at most N of the wave's memory operations are outstanding (they finish in order).
template <int N>
__device__ inline void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  // vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]; the other counters unconstrained
  __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}
// The same for a number known at run time only (the same in all lanes), up to kMost.
template <int kMost>
__device__ inline void wait_loads_at_most(int n) {
  if constexpr (kMost == 0) {
    wait_loads<0>();
  } else {
    if (n >= kMost) wait_loads<kMost>();
    else wait_loads_at_most<kMost - 1>(n);
  }
}

}  // namespace bc4g
