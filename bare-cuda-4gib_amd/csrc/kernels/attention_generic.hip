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
//
// A tile's keys, and then its values, pass through LDS 64 dimensions at a time, so that memory is read along its
// rows (a key's dimensions side by side; a dimension's tokens side by side: values are kept transposed) and the
// arithmetic reads LDS without bank conflicts: lane = key for the scores, lane = dimension for the output.  Read
// straight from memory with a key to a lane, every load touched 64 lines (a 2,048-token prompt of the 32-bit path at
// TinyLlama's sizes: 16.4 ms a layer in this kernel, four fifths of the prompt's time).  A score is still the sum over
// the dimensions in ascending order in one lane, and an output the sum over the keys in ascending order: the same
// bits as before.
#include <float.h>
#include <math.h>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kMaxHeadDim = 256;
constexpr int kDimsPerLane = kMaxHeadDim / kWave;
constexpr int kTilePad = kWave + 1;          // a tile's row in LDS: 64 floats and one, so that a column is 64 banks

__device__ inline float4 load_four(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ inline float4 load_four(const bf16_t* p) {
  const uint2 bits = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(bits.x << 16), __uint_as_float(bits.x & 0xffff0000u),
                     __uint_as_float(bits.y << 16), __uint_as_float(bits.y & 0xffff0000u));
}

template <typename T>
__global__ __launch_bounds__(kWave) void attention_generic_kernel(
    const T* __restrict__ qkv, T* __restrict__ out, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ positions, int n_heads,
    int n_kv_heads, int head_dim, int page_tokens, int window, float scale, int q_stride) {
  __shared__ float q_s[kMaxHeadDim];
  __shared__ float p_s[kWave];
  __shared__ float tile[kWave][kTilePad];      // keys: [key][dimension]; values: [key][dimension] too
  const int row = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int kvh = head / (n_heads / n_kv_heads);
  const int pos = positions[row];
  const int32_t* table = block_table + static_cast<long>(row_seq[row]) * table_stride;
  const long qkv_stride = q_stride;
  const T* q = qkv + row * qkv_stride + static_cast<long>(head) * head_dim;
  for (int c = lane; c < head_dim; c += kWave) q_s[c] = to_float(q[c]);
  __syncthreads();

  const int first = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // four dimensions of a key as one load, where every such group is aligned
  const bool by_four = head_dim % 4 == 0 && reinterpret_cast<uintptr_t>(k_cache) % (4 * sizeof(T)) == 0;
  float m = -INFINITY, l = 0.f;
  float acc[kDimsPerLane];
#pragma unroll
  for (int i = 0; i < kDimsPerLane; ++i) acc[i] = 0.f;

  for (int j0 = first; j0 <= pos; j0 += kWave) {
    const int n_here = min(kWave, pos - j0 + 1);
    const int j = j0 + lane;
    const bool seen = j <= pos;
    // scores: lane = key, the dimensions 64 at a time through the tile
    float dot = 0.f;
    for (int c0 = 0; c0 < head_dim; c0 += kWave) {
      const int width = min(kWave, head_dim - c0);
      // A key's dimensions side by side.  The loads of a tile are asked for together and written to LDS afterwards:
      // one after the other, each waiting for the last, a lone wave (a decode step) would pay 64 ways to memory a tile.
      if (by_four) {                                         // four dimensions a lane, four keys a load
        const int quad = (lane % 16) * 4, sub = lane / 16;
        float4 held[16];
#pragma unroll
        for (int b = 0; b < 16; ++b) {
          const int jk = j0 + b * 4 + sub;
          held[b] = make_float4(0.f, 0.f, 0.f, 0.f);
          if (jk <= pos && quad < width) {
            const long page = table[jk / page_tokens];
            held[b] = load_four(k_cache + ((page * n_kv_heads + kvh) * page_tokens + jk % page_tokens) * head_dim +
                                c0 + quad);
          }
        }
#pragma unroll
        for (int b = 0; b < 16; ++b) {
          float* to = &tile[b * 4 + sub][quad];
          to[0] = held[b].x, to[1] = held[b].y, to[2] = held[b].z, to[3] = held[b].w;
        }
      } else {                                               // lane = dimension, eight keys asked for together
        for (int jb = 0; jb < n_here; jb += 8) {
          float held[8];
#pragma unroll
          for (int b = 0; b < 8; ++b) {
            const int jk = j0 + jb + b;
            held[b] = 0.f;
            if (jk <= pos && lane < width) {
              const long page = table[jk / page_tokens];
              held[b] = to_float(k_cache[((page * n_kv_heads + kvh) * page_tokens + jk % page_tokens) * head_dim +
                                         c0 + lane]);
            }
          }
#pragma unroll
          for (int b = 0; b < 8; ++b) tile[jb + b][lane] = held[b];
        }
      }
      __syncthreads();
      if (seen)
        for (int c = 0; c < width; ++c) dot = fmaf(q_s[c0 + c], tile[lane][c], dot);
      __syncthreads();
    }
    const float s = seen ? dot * scale : -INFINITY;
    const float m_new = fmaxf(m, wave_max(s));  // finite: key j0 is always visible
    const float p = seen ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);         // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
    p_s[lane] = p;
#pragma unroll
    for (int i = 0; i < kDimsPerLane; ++i) acc[i] *= alpha;
    // output: the tile's values 64 dimensions at a time; a dimension's tokens lie side by side in a page, so lane =
    // key for the reading, and lane = dimension for the sums over the keys in ascending order
    const long v_page = seen ? table[j / page_tokens] : 0;
    const T* vkey = v_cache + (v_page * n_kv_heads + kvh) * head_dim * page_tokens + j % page_tokens;
#pragma unroll
    for (int i = 0; i < kDimsPerLane; ++i) {
      const int c0 = i * kWave;
      if (c0 >= head_dim) break;
      const int width = min(kWave, head_dim - c0);
      for (int cb = 0; cb < width; cb += 8) {              // eight dimensions asked for together
        float held[8];
#pragma unroll
        for (int b = 0; b < 8; ++b)
          held[b] = (seen && cb + b < width) ? to_float(vkey[static_cast<long>(c0 + cb + b) * page_tokens]) : 0.f;
#pragma unroll
        for (int b = 0; b < 8; ++b) tile[lane][cb + b] = held[b];
      }
      __syncthreads();
      if (lane < width)
        for (int jj = 0; jj < n_here; ++jj) acc[i] = fmaf(p_s[jj], tile[jj][lane], acc[i]);
      __syncthreads();
    }
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
