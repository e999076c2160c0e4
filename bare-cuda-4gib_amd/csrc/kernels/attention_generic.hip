// Causal softmax attention over the paged cache for any head size up to 256,
// any head counts, float or bfloat16 storage, in plain float arithmetic.  One
// wave per (query row, head): the attention of the 32-bit path and the fallback
// where the MFMA kernels refuse a size.  Prompt portions and single decoded
// tokens are the same to it: every row carries its request and its position.
//
// Keys are walked in ascending order in tiles of 64 with a running maximum and
// running sum (online softmax), so scores are never written to memory.  A row
// reads keys max(0, p - window + 1) .. p and nothing else: pages past its
// position, or before its window, may belong to nobody.
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kMaxHeadDim = 256;
constexpr int kDimsPerLane = kMaxHeadDim / kWave;

template <typename T>
__global__ __launch_bounds__(kWave) void attention_generic_kernel(
    const T* __restrict__ qkv, T* __restrict__ out, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions, int n_heads,
    int n_kv_heads, int head_dim, int page_tokens, int window, float scale, int q_stride) {
  __shared__ float q_s[kMaxHeadDim];
  __shared__ float p_s[kWave];
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int kvh = head / (n_heads / n_kv_heads);
  const int pos = positions[row];
  const int32_t* table = block_table + static_cast<long>(row_seq[row]) * table_stride;
  const long qkv_stride = q_stride;
  const T* q = qkv + row * qkv_stride + static_cast<long>(head) * head_dim;
  for (int c = lane; c < head_dim; c += kWave) q_s[c] = to_float(q[c]);
  __syncthreads();

  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[kDimsPerLane];
#pragma unroll
  for (int i = 0; i < kDimsPerLane; ++i) acc[i] = 0.f;

  for (int j0 = first; j0 <= pos; j0 += kWave) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= pos) {
      const long page = table[j / page_tokens];
      const T* krow = k_cache + ((page * n_kv_heads + kvh) * page_tokens + j % page_tokens) * head_dim;
      float dot = 0.f;
      for (int c = 0; c < head_dim; ++c) dot = fmaf(q_s[c], to_float(krow[c]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: key j0 is always visible
    const float p = (j <= pos) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);         // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kDimsPerLane; ++i) acc[i] *= alpha;
    const int n_here = min(kWave, pos - j0 + 1);
    for (int jj = 0; jj < n_here; ++jj) {
      const int jk = j0 + jj;
      const long page = table[jk / page_tokens];
      const T* vcol = v_cache + (page * n_kv_heads + kvh) * head_dim * page_tokens + jk % page_tokens;
      const float pj = p_s[jj];
#pragma unroll
      for (int i = 0; i < kDimsPerLane; ++i) {
        const int c = lane + i * kWave;
        if (c < head_dim) acc[i] = fmaf(pj, to_float(vcol[static_cast<long>(c) * page_tokens]), acc[i]);
      }
    }
    __syncthreads();
  }
  const float inv_l = 1.0f / l;
  T* o = out + (static_cast<long>(row) * n_heads + head) * head_dim;
#pragma unroll
  for (int i = 0; i < kDimsPerLane; ++i) {
    const int c = lane + i * kWave;
    if (c < head_dim) o[c] = from_float<T>(acc[i] * inv_l);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_attention_generic(const void* qkv, int q_stride, void* out, int dtype, const void* k_cache,
                                      const void* v_cache, const int32_t* block_table, int table_stride,
                                      const int32_t* row_seq, const int32_t* positions, int n_tokens,
                                      int n_heads, int n_kv_heads, int head_dim, int page_tokens,
                                      int num_pages, int window, float scale, void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0,
               "attention: bad sizes T=%d heads=%d/%d", n_tokens, n_heads, n_kv_heads);
  BC4G_REQUIRE(head_dim > 0 && head_dim <= kMaxHeadDim, "attention: head_dim %d is beyond %d", head_dim,
               kMaxHeadDim);
  BC4G_REQUIRE(page_tokens > 0 && num_pages > 0 && table_stride > 0 && window >= 0,
               "attention: bad cache sizes page_tokens=%d pages=%d table_stride=%d window=%d", page_tokens,
               num_pages, table_stride, window);
  BC4G_REQUIRE(n_heads <= 65535, "attention: %d heads are beyond the grid limit", n_heads);
  BC4G_REQUIRE(q_stride >= n_heads * head_dim, "attention: bad query row stride %d", q_stride);
  if (n_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(n_tokens, n_heads);
  if (dtype == kF32) {
    attention_generic_kernel<float><<<grid, kWave, 0, s>>>(
        static_cast<const float*>(qkv), static_cast<float*>(out), static_cast<const float*>(k_cache),
        static_cast<const float*>(v_cache), block_table, table_stride, row_seq, positions, n_heads,
        n_kv_heads, head_dim, page_tokens, window, scale, q_stride);
  } else if (dtype == kBF16) {
    attention_generic_kernel<bf16_t><<<grid, kWave, 0, s>>>(
        static_cast<const bf16_t*>(qkv), static_cast<bf16_t*>(out), static_cast<const bf16_t*>(k_cache),
        static_cast<const bf16_t*>(v_cache), block_table, table_stride, row_seq, positions, n_heads,
        n_kv_heads, head_dim, page_tokens, window, scale, q_stride);
  } else {
    return fail("attention: unknown dtype %d", dtype);
  }
  return check_launch("attention_generic");
}
