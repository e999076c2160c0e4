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
  // The LDS base of a wave-wide load travels in m0, which the compiler also uses for purposes of its own (it
  // sets it right before each): the statement sets m0 and uses it at once, and says that it clobbers it.  The
  // compiler does not know the instruction, so the waits for it are written by hand (wait_loads): between asking
  // and waiting a loop must hold no other vector-memory operation of the wave -- no spill, nothing the compiler
  // might add -- or the hand-counted waits count the wrong loads.
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(global), "s"(lds_address) : "memory", "m0");
}

// The same from one base address for the whole wave (in scalar registers) plus each lane's offset in bytes.
__device__ inline void load_to_lds_16(const void* wave_base, unsigned lane_offset, unsigned lds_address) {
  // (the base is the same in every lane; said so, half by half, it is kept in scalar registers)
  const uintptr_t bits = reinterpret_cast<uintptr_t>(wave_base);
  const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits));
  const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits >> 32));
  wave_base = reinterpret_cast<const void*>((static_cast<uintptr_t>(hi) << 32) | lo);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(wave_base), "s"(lds_address)
               : "memory", "m0");
}

// Several such loads to one stretch of LDS as ONE statement: N chunks of 1 KB side by side, chunk r from bases[r]
// (the same in every lane) plus each lane's offset in bytes.  The LDS address is set once, to the chunk in the
// middle of the stretch, and each load adds its (r - N / 2) * 1024 bytes to it through the instruction's offset
// field -- and to its memory address, so that much is taken off the base here.  (Setting the LDS address anew for
// every load costs the wave hundreds of clocks a load: the write to m0 waits for the load before it, which still
// needs the old value.)  The write to m0 and the loads that rely on it stand in one asm statement that says it
// clobbers m0, so nothing the compiler makes of the code around them -- indexing a register array at run time
// writes m0 on this hardware -- can come between them.
template <int N>
__device__ inline void load_chunks_to_lds(const void* const (&bases)[N], unsigned lane_offset, unsigned lds_first_chunk) {
  static_assert(N == 1 || N == 2 || N == 4 || N == 8, "chunks a wave brings");
  constexpr int kMid = N / 2;
  const void* b[N];
#pragma unroll
  for (int r = 0; r < N; ++r) {
    const uintptr_t bits = reinterpret_cast<uintptr_t>(bases[r]) - (r - kMid) * 1024;
    const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits));
    const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(bits >> 32));
    b[r] = reinterpret_cast<const void*>((static_cast<uintptr_t>(hi) << 32) | lo);
  }
  const unsigned mid = __builtin_amdgcn_readfirstlane(lds_first_chunk + kMid * 1024);
#define BC4G_LDS_LOAD(i, op) "global_load_lds_dwordx4 %1, %" #op " offset:" #i "\n\t"
  if constexpr (N == 1) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" BC4G_LDS_LOAD(0, 2)
                 ::"s"(mid), "v"(lane_offset), "s"(b[0]) : "memory", "m0");
  } else if constexpr (N == 2) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" BC4G_LDS_LOAD(-1024, 2) BC4G_LDS_LOAD(0, 3)
                 ::"s"(mid), "v"(lane_offset), "s"(b[0]), "s"(b[1]) : "memory", "m0");
  } else if constexpr (N == 4) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" BC4G_LDS_LOAD(-2048, 2) BC4G_LDS_LOAD(-1024, 3) BC4G_LDS_LOAD(0, 4)
                 BC4G_LDS_LOAD(1024, 5)
                 ::"s"(mid), "v"(lane_offset), "s"(b[0]), "s"(b[1]), "s"(b[2]), "s"(b[3]) : "memory", "m0");
  } else {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t" BC4G_LDS_LOAD(-4096, 2) BC4G_LDS_LOAD(-3072, 3) BC4G_LDS_LOAD(-2048, 4)
                 BC4G_LDS_LOAD(-1024, 5) BC4G_LDS_LOAD(0, 6) BC4G_LDS_LOAD(1024, 7) BC4G_LDS_LOAD(2048, 8)
                 BC4G_LDS_LOAD(3072, 9)
                 ::"s"(mid), "v"(lane_offset), "s"(b[0]), "s"(b[1]), "s"(b[2]), "s"(b[3]), "s"(b[4]), "s"(b[5]), "s"(b[6]),
                 "s"(b[7]) : "memory", "m0");
  }
#undef BC4G_LDS_LOAD
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
