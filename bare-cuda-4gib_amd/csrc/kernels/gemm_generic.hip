// out[m, n] (+)= sum_k a[m, k] * w[n, k] for any sizes and any mix of float and
// bfloat16 operands, in plain float FMA (no matrix cores): the matrix product
// of the 32-bit path, and the fallback where the MFMA kernels refuse a size.
//
// Each output element is the sum over k in ascending order in one thread, so
// a row's result does not depend on how many rows the call has -- nor on which of the
// two tile sizes below serves the call: 64 x 64 outputs a block (four by four a thread),
// or, for up to 16 rows (a decode step), 16 x 16 (one a thread, k staged 64 at a time),
// which brings sixteen times the blocks to stream the weights of a product with few rows
// (a decode step of the 32-bit path at TinyLlama's sizes: 43 ms with the large tile alone).
#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kFewRows = 16;   // rows up to which the small tile serves

template <typename TA, typename TW, typename TO, bool kAccumulate, int kPerThread, int kStepK>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ a,
                                                           const TW* __restrict__ w,
                                                           TO* __restrict__ out, int m, int n, int k) {
  constexpr int kTile = 16 * kPerThread;   // output tile per block, both ways
  // k-major tiles, padded so that the 16 threads of a row group hit different banks.
  __shared__ float as[kStepK][kTile + 1];
  __shared__ float ws[kStepK][kTile + 1];
  const int tx = threadIdx.x % 16;  // columns tx*kPerThread ..
  const int ty = threadIdx.x / 16;  // rows    ty*kPerThread ..
  const long m0 = static_cast<long>(blockIdx.y) * kTile;
  const long n0 = static_cast<long>(blockIdx.x) * kTile;

  float acc[kPerThread][kPerThread];
#pragma unroll
  for (int i = 0; i < kPerThread; ++i)
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) acc[i][j] = 0.f;

  // A step's operands are asked for a step ahead, into registers, so that the way from memory lies beside the step
  // before's arithmetic instead of before its own: kTile rows x kStepK k elements per operand, the same number a
  // thread; k fastest for coalescing.
  constexpr int kLoads = kTile * kStepK / 256;
  float ar[kLoads], wr[kLoads];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int r = 0; r < kLoads; ++r) {
      const int e = threadIdx.x + r * 256;
      const int kk = e % kStepK, row = e / kStepK;
      const long gm = m0 + row, gn = n0 + row;
      const int gk = k0 + kk;
      ar[r] = (gm < m && gk < k) ? to_float(a[gm * k + gk]) : 0.f;
      wr[r] = (gn < n && gk < k) ? to_float(w[gn * k + gk]) : 0.f;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < k; k0 += kStepK) {
#pragma unroll
    for (int r = 0; r < kLoads; ++r) {
      const int e = threadIdx.x + r * 256;
      as[e % kStepK][e / kStepK] = ar[r];
      ws[e % kStepK][e / kStepK] = wr[r];
    }
    __syncthreads();
    if (k0 + kStepK < k) fetch(k0 + kStepK);
#pragma unroll
    for (int kk = 0; kk < kStepK; ++kk) {
      float av[kPerThread], wv[kPerThread];
#pragma unroll
      for (int i = 0; i < kPerThread; ++i) av[i] = as[kk][ty * kPerThread + i];
#pragma unroll
      for (int j = 0; j < kPerThread; ++j) wv[j] = ws[kk][tx * kPerThread + j];
#pragma unroll
      for (int i = 0; i < kPerThread; ++i)
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < kPerThread; ++i) {
    const long gm = m0 + ty * kPerThread + i;
    if (gm >= m) continue;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
      const long gn = n0 + tx * kPerThread + j;
      if (gn >= n) continue;
      if constexpr (kAccumulate) {
        out[gm * n + gn] = from_float<TO>(to_float(out[gm * n + gn]) + acc[i][j]);
      } else {
        out[gm * n + gn] = from_float<TO>(acc[i][j]);
      }
    }
  }
}

template <typename TA, typename TW, typename TO, bool kAcc>
void launch(const void* a, const void* w, void* out, int m, int n, int k, hipStream_t s) {
  if (m <= kFewRows) {
    gemm_generic_kernel<TA, TW, TO, kAcc, 1, 64><<<dim3(ceil_div(n, 16), 1), 256, 0, s>>>(
        static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out), m, n, k);
    return;
  }
  gemm_generic_kernel<TA, TW, TO, kAcc, 4, 16><<<dim3(ceil_div(n, 64), ceil_div(m, 64)), 256, 0, s>>>(
      static_cast<const TA*>(a), static_cast<const TW*>(w), static_cast<TO*>(out), m, n, k);
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_gemm_generic(const void* a, int a_dtype, const void* w, int w_dtype, void* out,
                                 int out_dtype, int accumulate, int m, int n, int k, void* stream) {
  BC4G_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm: bad sizes M=%d N=%d K=%d", m, n, k);
  BC4G_REQUIRE(!accumulate || out_dtype == kF32, "gemm: accumulation needs a float32 output");
  BC4G_REQUIRE(ceil_div(m, 64) <= 65535, "gemm: M=%d is beyond the grid limit", m);
  if (m == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int key = a_dtype * 100 + w_dtype * 10 + out_dtype;
  switch (key) {
    case 0:   // f32 x f32 -> f32
      if (accumulate) launch<float, float, float, true>(a, w, out, m, n, k, s);
      else launch<float, float, float, false>(a, w, out, m, n, k, s);
      break;
    case 110:  // bf16 x bf16 -> f32
      if (accumulate) launch<bf16_t, bf16_t, float, true>(a, w, out, m, n, k, s);
      else launch<bf16_t, bf16_t, float, false>(a, w, out, m, n, k, s);
      break;
    case 111:  // bf16 x bf16 -> bf16
      launch<bf16_t, bf16_t, bf16_t, false>(a, w, out, m, n, k, s);
      break;
    case 100:  // bf16 x f32 -> f32
      if (accumulate) launch<bf16_t, float, float, true>(a, w, out, m, n, k, s);
      else launch<bf16_t, float, float, false>(a, w, out, m, n, k, s);
      break;
    case 101:  // bf16 x f32 -> bf16
      launch<bf16_t, float, bf16_t, false>(a, w, out, m, n, k, s);
      break;
    default:
      return fail("gemm: unsupported dtypes a=%d w=%d out=%d", a_dtype, w_dtype, out_dtype);
  }
  return check_launch("gemm_generic");
}
