// Shared device helpers for the gfx950 kernels: storage types, wave64
// reductions, error reporting of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bc4g {

constexpr int kWave = 64;  // CDNA wavefront width

// A workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads() also waits for
// every global load the wave has in flight, which undoes a prefetch; here those loads stay in flight
// (the compiler still waits for a load's data where it is used).
__device__ inline void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- storage types ---------------------------------------------------------
// Activations, weights and cache are float or bfloat16; bfloat16 is handled as
// its 16-bit pattern and widened/rounded by hand so that every kernel states
// where it rounds.  All arithmetic is float.
struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float to_float(float v) { return v; }
__host__ __device__ inline float to_float(bf16_t v) {
  union { uint32_t u; float f; } c;
  c.u = static_cast<uint32_t>(v.bits) << 16;
  return c.f;
}

// Round to nearest, ties to even; NaN stays NaN.
__host__ __device__ inline uint16_t bf16_bits_from_float(float f) {
  union { uint32_t u; float f; } c;
  c.f = f;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((c.u >> 16) | 0x0040u);
  const uint32_t lsb = (c.u >> 16) & 1u;
  c.u += 0x7fffu + lsb;
  return static_cast<uint16_t>(c.u >> 16);
}

template <typename T> __host__ __device__ inline T from_float(float f);
template <> __host__ __device__ inline float from_float<float>(float f) { return f; }
template <> __host__ __device__ inline bf16_t from_float<bf16_t>(float f) {
  bf16_t r;
  r.bits = bf16_bits_from_float(f);
  return r;
}

// ---- the key/value cache in fragment order -----------------------------------
// A bfloat16 cache whose head size (16 .. 256) and page size are multiples of 16 -- the caches the
// matrix-core attention kernel reads -- keeps the elements of every (page, key/value head) region of
// page_tokens * head_dim elements in the order in which that kernel's lanes take them, one block of
// 16 tokens after the other:
//   keys    [token / 16][dim / 8][token % 16][dim % 8]
//           the A operand of the scores for 16 keys x 32 dims (lane l: key l % 16, dims 8 * (l / 16) ..)
//           is 1 KB that the 64 lanes read in lane order
//   values  [token / 16][dim / 16][(token % 16) / 4][dim % 16][token % 4]
//           the A operand of the output for 16 dims x 16 keys (lane l: dim l % 16, keys 4 * (l / 16) ..)
//           is 512 bytes in lane order
// Every other cache (float, other sizes) is plain: keys [token][dim], values [dim][token].
__host__ __device__ inline bool cache_fragment_order(bool is_bf16, int head_dim, int page_tokens) {
  return is_bf16 && head_dim % 16 == 0 && head_dim >= 16 && head_dim <= 256 && page_tokens % 16 == 0;
}
__host__ __device__ inline long frag_k_offset(int token, int dim, int head_dim) {
  return static_cast<long>(token / 16) * (16 * head_dim) + ((dim / 8) * 16 + token % 16) * 8 + dim % 8;
}
__host__ __device__ inline long frag_v_offset(int token, int dim, int head_dim) {
  return static_cast<long>(token / 16) * (16 * head_dim) + (((dim / 16) * 4 + (token % 16) / 4) * 16 + dim % 16) * 4 +
         token % 4;
}

// ---- wave64 / block reductions --------------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds at least 16 floats.
// Every thread gets the result.  The order of additions depends only on the
// block size, so a row's result does not depend on what else is in the batch.
__device__ inline float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}
__device__ inline float block_max(float v, float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int nwaves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float m = scratch[0];
  for (int w = 1; w < nwaves; ++w) m = fmaxf(m, scratch[w]);
  return m;
}

// ---- host side --------------------------------------------------------------
enum DType : int { kF32 = 0, kBF16 = 1 };

// Records a message for bc4g_last_error() and returns a non-zero status.
int fail(const char* fmt, ...);
int check_launch(const char* what);
int compute_units();   // of the current device (256 if it cannot be asked)

inline int ceil_div(long a, long b) { return static_cast<int>((a + b - 1) / b); }

}  // namespace bc4g

#define BC4G_REQUIRE(cond, ...)                  \
  do {                                           \
    if (!(cond)) return bc4g::fail(__VA_ARGS__); \
  } while (0)
