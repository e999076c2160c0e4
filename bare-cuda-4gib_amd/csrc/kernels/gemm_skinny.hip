// out[m, n] = sum_k x[m, k] * w[n, k] for few rows m (a decode step: m <= 64), bfloat16 operands.
//
// The weights are read once, straight from memory into matrix-core registers: a workgroup owns
// 16 output columns n (16 rows of w) and all of k; its 8 waves split k between them, each wave
// feeding 16x16x32 MFMAs with w as the A operand (16-byte loads, rows of w are contiguous in k)
// and x as the B operand (x is small and comes from cache).  The waves' partial sums meet in
// LDS and are added in wave order, so a result does not depend on the number of rows or on
// timing.  The epilogue stores bfloat16 or float, adds into the float residual stream, or, when
// w holds gate rows followed by up rows, applies SwiGLU to the pair of sums.
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kWaves = 8;
constexpr int kUnroll = 4;       // MFMA k-steps (of 32) whose loads are issued together
constexpr int kRedPad = 17;

enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAccumF32 = 2, kSwigluBf16 = 3 };

template <int MT, int EPI>
__global__ __launch_bounds__(kWaves * kWave) void gemm_skinny_kernel(const bf16_t* __restrict__ x,
                                                                     const bf16_t* __restrict__ w,
                                                                     void* __restrict__ out, int m, int n,
                                                                     int k, int n_out) {
  constexpr int kSets = (EPI == kSwigluBf16) ? 2 : 1;   // gate and up rows
  __shared__ float red[kWaves][kSets][MT][16][kRedPad];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int col = lane % 16, grp = lane / 16;
  const int n0 = blockIdx.x * 16;

  const int chunk = ((k + kWaves * 32 - 1) / (kWaves * 32)) * 32;
  const int k_begin = wave * chunk;
  const int k_end = min(k, k_begin + chunk);

  floatx4 acc[kSets][MT];
#pragma unroll
  for (int s = 0; s < kSets; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[s][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int wrow = n0 + col;                           // this lane's row of w (output column)
  const bool wrow_ok = wrow < n_out;
  const bf16_t* wptr[kSets];
#pragma unroll
  for (int s = 0; s < kSets; ++s) wptr[s] = w + (static_cast<long>(wrow) + static_cast<long>(s) * n_out) * k;

  for (int k0 = k_begin; k0 < k_end; k0 += 32 * kUnroll) {
    uint4 wv[kSets][kUnroll], xv[MT][kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int kk = k0 + 32 * u + 8 * grp;
      const bool ok = kk < k_end;
#pragma unroll
      for (int s = 0; s < kSets; ++s) wv[s][u] = (ok && wrow_ok) ? load16(wptr[s] + kk) : zero16();
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int row = t * 16 + col;
        xv[t][u] = (ok && row < m) ? load16(x + static_cast<long>(row) * k + kk) : zero16();
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
#pragma unroll
      for (int s = 0; s < kSets; ++s)
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[s][t] = mfma_16x16x32(wv[s][u], xv[t][u], acc[s][t]);
  }

  // acc[s][t][r] is the partial sum for output column n0 + 4*grp + r and row t*16 + col
#pragma unroll
  for (int s = 0; s < kSets; ++s)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][s][t][4 * grp + r][col] = acc[s][t][r];
  __syncthreads();

  for (int idx = threadIdx.x; idx < MT * 256; idx += kWaves * kWave) {
    const int nl = idx % 16, row = idx / 16;
    const int gn = n0 + nl;
    if (row >= m || gn >= n_out) continue;
    float sum[kSets];
#pragma unroll
    for (int s = 0; s < kSets; ++s) {
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < kWaves; ++wv) v += red[wv][s][row / 16][nl][row % 16];
      sum[s] = v;
    }
    const long o = static_cast<long>(row) * n_out + gn;
    if constexpr (EPI == kStoreBf16) {
      static_cast<bf16_t*>(out)[o] = from_float<bf16_t>(sum[0]);
    } else if constexpr (EPI == kStoreF32) {
      static_cast<float*>(out)[o] = sum[0];
    } else if constexpr (EPI == kAccumF32) {
      static_cast<float*>(out)[o] += sum[0];
    } else {
      const float g = sum[0], u = sum[kSets - 1];
      static_cast<bf16_t*>(out)[o] = from_float<bf16_t>((g / (1.0f + expf(-g))) * u);
    }
  }
}

template <int EPI>
int launch(const void* x, const void* w, void* out, int m, int n, int k, int n_out, hipStream_t s) {
  const int mt = (m + 15) / 16;
  dim3 grid((n_out + 15) / 16), block(kWaves * kWave);
  const bf16_t* xp = static_cast<const bf16_t*>(x);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  switch (mt) {
    case 1: gemm_skinny_kernel<1, EPI><<<grid, block, 0, s>>>(xp, wp, out, m, n, k, n_out); break;
    case 2: gemm_skinny_kernel<2, EPI><<<grid, block, 0, s>>>(xp, wp, out, m, n, k, n_out); break;
    case 3: gemm_skinny_kernel<3, EPI><<<grid, block, 0, s>>>(xp, wp, out, m, n, k, n_out); break;
    case 4: gemm_skinny_kernel<4, EPI><<<grid, block, 0, s>>>(xp, wp, out, m, n, k, n_out); break;
    default: return fail("gemm_skinny: M=%d is beyond 64 rows", m);
  }
  return check_launch("gemm_skinny");
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_gemm_skinny(const void* x, const void* w, void* out, int epilogue, int m, int n, int k,
                                void* stream) {
  BC4G_REQUIRE(m >= 0 && m <= 64, "gemm_skinny: M=%d must be at most 64", m);
  BC4G_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "gemm_skinny: K=%d must be a positive multiple of 8 (N=%d)", k, n);
  BC4G_REQUIRE(epilogue != kSwigluBf16 || n % 2 == 0, "gemm_skinny: SwiGLU needs gate and up rows, N=%d is odd", n);
  if (m == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (epilogue) {
    case kStoreBf16: return launch<kStoreBf16>(x, w, out, m, n, k, n, s);
    case kStoreF32: return launch<kStoreF32>(x, w, out, m, n, k, n, s);
    case kAccumF32: return launch<kAccumF32>(x, w, out, m, n, k, n, s);
    case kSwigluBf16: return launch<kSwigluBf16>(x, w, out, m, n, k, n / 2, s);
    default: return fail("gemm_skinny: unknown epilogue %d", epilogue);
  }
}
