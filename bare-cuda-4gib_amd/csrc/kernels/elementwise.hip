// Embedding gather, RMSNorm, SwiGLU, rotary positions + cache write, argmax
// and sampling.  One instantiation per storage type; all arithmetic in float.
#include <float.h>
#include <math.h>

#include <mutex>

#include "api.h"
#include "no_alloc.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kBlock = 256;

// ---- embedding -------------------------------------------------------------
template <typename TT>
__global__ void embed_gather_kernel(const TT* __restrict__ table, const int32_t* __restrict__ ids,
                                    float* __restrict__ out, int hidden) {
  const size_t row = blockIdx.x;
  const TT* src = table + static_cast<size_t>(ids[row]) * hidden;
  float* dst = out + row * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]);
}

// ---- RMSNorm ---------------------------------------------------------------
// eps is added to the mean square; sum and rsqrt in float.
template <typename TW, typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                               const TW* __restrict__ w, TO* __restrict__ out, int hidden, float eps) {
  __shared__ float scratch[16];
  const size_t src_row = rows ? static_cast<size_t>(rows[blockIdx.x]) : blockIdx.x;
  const float* xr = x + src_row * hidden;
  TO* orow = out + static_cast<size_t>(blockIdx.x) * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = xr[i];
    ss += v * v;
  }
  const float mean_sq = block_sum(ss, scratch) / static_cast<float>(hidden);
  const float scale = 1.0f / sqrtf(mean_sq + eps);
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    orow[i] = from_float<TO>(xr[i] * scale * to_float(w[i]));
  }
}

// The same for widths that are a multiple of 8 and at most 256 * 8 * CHUNKS: a thread keeps its
// elements (CHUNKS pieces of 8) in registers between the sum and the scaling -- the row is read
// once, in 16-byte pieces, and written in 16-byte (bfloat16) or 32-byte pieces.
template <typename TW, typename TO, int CHUNKS>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows,
                                                           const TW* __restrict__ w, TO* __restrict__ out, int hidden,
                                                           float eps) {
  __shared__ float scratch[16];
  const size_t src_row = rows ? static_cast<size_t>(rows[blockIdx.x]) : blockIdx.x;
  const float* xr = x + src_row * hidden;
  TO* orow = out + static_cast<size_t>(blockIdx.x) * hidden;
  float v[CHUNKS][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i < hidden) {
      const float4 a = *reinterpret_cast<const float4*>(xr + i), b = *reinterpret_cast<const float4*>(xr + i + 4);
      v[c][0] = a.x; v[c][1] = a.y; v[c][2] = a.z; v[c][3] = a.w;
      v[c][4] = b.x; v[c][5] = b.y; v[c][6] = b.z; v[c][7] = b.w;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][e] = 0.f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[c][e] * v[c][e];
  }
  const float mean_sq = block_sum(ss, scratch) / static_cast<float>(hidden);
  const float scale = 1.0f / sqrtf(mean_sq + eps);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i >= hidden) continue;
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = v[c][e] * scale * to_float(w[i + e]);
    if constexpr (sizeof(TO) == 2) {
      uint32_t pk[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        pk[e] = static_cast<uint32_t>(bf16_bits_from_float(y[2 * e])) | (static_cast<uint32_t>(bf16_bits_from_float(y[2 * e + 1])) << 16);
      *reinterpret_cast<uint4*>(orow + i) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) orow[i + e] = from_float<TO>(y[e]);
    }
  }
}

// The same for a stream whose last addition is still in parts: x += parts[0] + parts[1] + ... (in that order, every
// part [n_rows, hidden] floats), x written back, then its norm -- what follows a product whose k was cut over
// workgroups (bc4g_gemm_mfma_parts).
template <typename TW, typename TO, int CHUNKS>
__global__ __launch_bounds__(256) void rmsnorm_sum_rows_kernel(float* __restrict__ x, const float* __restrict__ parts, int n_parts,
                                                               const TW* __restrict__ w, TO* __restrict__ out, int n_rows,
                                                               int hidden, float eps) {
  __shared__ float scratch[16];
  const size_t at = static_cast<size_t>(blockIdx.x) * hidden, part_stride = static_cast<size_t>(n_rows) * hidden;
  float* xr = x + at;
  TO* orow = out + at;
  float v[CHUNKS][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i < hidden) {
      float4 a = *reinterpret_cast<const float4*>(xr + i), b = *reinterpret_cast<const float4*>(xr + i + 4);
      for (int p = 0; p < n_parts; ++p) {
        const float* pr = parts + p * part_stride + at + i;
        const float4 pa = *reinterpret_cast<const float4*>(pr), pb = *reinterpret_cast<const float4*>(pr + 4);
        a.x += pa.x; a.y += pa.y; a.z += pa.z; a.w += pa.w;
        b.x += pb.x; b.y += pb.y; b.z += pb.z; b.w += pb.w;
      }
      *reinterpret_cast<float4*>(xr + i) = a;
      *reinterpret_cast<float4*>(xr + i + 4) = b;
      v[c][0] = a.x; v[c][1] = a.y; v[c][2] = a.z; v[c][3] = a.w;
      v[c][4] = b.x; v[c][5] = b.y; v[c][6] = b.z; v[c][7] = b.w;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][e] = 0.f;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[c][e] * v[c][e];
  }
  const float mean_sq = block_sum(ss, scratch) / static_cast<float>(hidden);
  const float scale = 1.0f / sqrtf(mean_sq + eps);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = (c * 256 + threadIdx.x) * 8;
    if (i >= hidden) continue;
    float y[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = v[c][e] * scale * to_float(w[i + e]);
    if constexpr (sizeof(TO) == 2) {
      uint32_t pk[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        pk[e] = static_cast<uint32_t>(bf16_bits_from_float(y[2 * e])) | (static_cast<uint32_t>(bf16_bits_from_float(y[2 * e + 1])) << 16);
      *reinterpret_cast<uint4*>(orow + i) = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) orow[i + e] = from_float<TO>(y[e]);
    }
  }
}

// ---- SwiGLU ----------------------------------------------------------------
// interleaved 0: a row of gu holds the gate values, then the up values.  1: blocks of 16 -- eight
// gate values followed by the eight up values of the same outputs (the layout the fused
// weight-streaming kernel produces and consumes).
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, long total, int inter,
                              int interleaved) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const long t = idx / inter;
    const int i = static_cast<int>(idx - t * inter);
    const long gi = interleaved ? (i / 8) * 16 + i % 8 : i;
    const long ui = interleaved ? gi + 8 : inter + i;
    const float g = to_float(gu[t * 2 * inter + gi]);
    const float u = to_float(gu[t * 2 * inter + ui]);
    out[idx] = from_float<T>((g / (1.0f + expf(-g))) * u);
  }
}

// ---- rotary positions + cache write -----------------------------------------
// One thread per (token, head among q|k|v, pair).  A pair is (i, i + rotary_dim/2)
// for i < rotary_dim/2; dimensions at or beyond rotary_dim pass through, handled
// by the threads with pair >= rotary_dim/2 as (lo = rotary_dim/2 + i .. ) below.
// block_pairs != 0: the head's dimensions were reordered in blocks of 16 (eight "lo" dimensions
// 8b .. 8b+7 followed by their partners), so pair i = 8b + t lies at 16b + t and 16b + 8 + t;
// this needs rotary_dim == head_dim or 0.
template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                     const int32_t* __restrict__ slot_map, T* __restrict__ k_cache,
                                     T* __restrict__ v_cache, long total, int n_heads, int n_kv_heads,
                                     int head_dim, int rotary_dim, float theta, int page_tokens,
                                     int write_kv, int block_pairs, int frag) {
  const int half = head_dim / 2;          // threads per head: each moves two elements
  const int rhalf = rotary_dim / 2;
  const int heads_total = n_heads + 2 * n_kv_heads;
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int j = static_cast<int>(idx % half);
    const long rest = idx / half;
    const int head = static_cast<int>(rest % heads_total);
    const long token = rest / heads_total;
    T* base = qkv + (token * heads_total + head) * head_dim;

    // Which two elements this thread owns: a rotated pair, or two pass-through elements.
    int i0, i1;
    bool rotate;
    if (block_pairs) {
      i0 = (j / 8) * 16 + j % 8;
      i1 = i0 + 8;
      rotate = rotary_dim > 0;
    } else if (j < rhalf) {
      i0 = j;
      i1 = j + rhalf;
      rotate = true;
    } else {
      i0 = rotary_dim + 2 * (j - rhalf);
      i1 = i0 + 1;
      rotate = false;
    }
    float a = to_float(base[i0]);
    float b = to_float(base[i1]);
    const bool is_v = head >= n_heads + n_kv_heads;
    if (rotate && !is_v) {
      float s, c;
      if constexpr (sizeof(T) == sizeof(float)) {
        // The 32-bit path works the angle out in double: a float angle carries an error of position * 2^-24
        // (1e-4 rad at position 2,000), which would show in the logits of long prompts as an error that grows with
        // the position, ten times what the rest of the path leaves, and hide what the path is there to show.
        const double inv_freq = 1.0 / pow(static_cast<double>(theta), (2.0 * j) / static_cast<double>(rotary_dim));
        double sd, cd;
        sincos(static_cast<double>(positions[token]) * inv_freq, &sd, &cd);
        s = static_cast<float>(sd);
        c = static_cast<float>(cd);
      } else {
        const float inv_freq = 1.0f / powf(theta, (2.0f * static_cast<float>(j)) / static_cast<float>(rotary_dim));
        sincosf(static_cast<float>(positions[token]) * inv_freq, &s, &c);
      }
      const float lo = a, hi = b;
      a = lo * c - hi * s;
      b = hi * c + lo * s;
    }
    if (head < n_heads) {
      base[i0] = from_float<T>(a);
      base[i1] = from_float<T>(b);
    } else if (write_kv) {
      const int kvh = is_v ? head - n_heads - n_kv_heads : head - n_heads;
      const int slot = slot_map[token];
      const long page = slot / page_tokens, off = slot % page_tokens;
      const long region = (page * n_kv_heads + kvh) * head_dim * page_tokens;
      if (frag) {  // the cache in fragment order
        T* dst = (is_v ? v_cache : k_cache) + region;
        const int o = static_cast<int>(off);
        dst[is_v ? frag_v_offset(o, i0, head_dim) : frag_k_offset(o, i0, head_dim)] = from_float<T>(a);
        dst[is_v ? frag_v_offset(o, i1, head_dim) : frag_k_offset(o, i1, head_dim)] = from_float<T>(b);
      } else if (is_v) {  // values are kept transposed: [page][kv head][dim][token]
        T* dst = v_cache + region + off;
        dst[static_cast<long>(i0) * page_tokens] = from_float<T>(a);
        dst[static_cast<long>(i1) * page_tokens] = from_float<T>(b);
      } else {     // keys: [page][kv head][token][dim]
        T* dst = k_cache + region + off * head_dim;
        dst[i0] = from_float<T>(a);
        dst[i1] = from_float<T>(b);
      }
    }
  }
}

// The angles of a step, once for all layers: table[token][i] = (cos, sin) of position * theta^(-2i/dim),
// i < dim/2, with the precise powf / sincosf of the kernel above.
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, float2* __restrict__ table, long total,
                                  int rhalf, float theta) {
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    const int i = static_cast<int>(idx % rhalf);
    const long token = idx / rhalf;
    const float inv_freq = 1.0f / powf(theta, (2.0f * static_cast<float>(i)) / static_cast<float>(2 * rhalf));
    float s, c;
    sincosf(static_cast<float>(positions[token]) * inv_freq, &s, &c);
    table[idx] = make_float2(c, s);
  }
}

// rope_kv_write for the block layout (block_pairs) with the step's table of angles: a thread takes
// one block of 16 elements -- pairs 8b .. 8b+7 of one head of one token -- with 16-byte loads and
// stores (values go to their pages element by element).  frag: the cache is in fragment order.
template <typename T>
__global__ void rope_kv_write_blocks_kernel(T* __restrict__ qkv, const float2* __restrict__ table,
                                            const int32_t* __restrict__ slot_map, T* __restrict__ k_cache,
                                            T* __restrict__ v_cache, long total, long n_tokens, int n_heads,
                                            int n_kv_heads, int head_dim, int rotate, int page_tokens, int write_kv,
                                            int frag) {
  const int blocks = head_dim / 16;
  const int heads_total = n_heads + 2 * n_kv_heads;
  const long stride = static_cast<long>(blockDim.x) * gridDim.x;
  // Items of the query heads first, a row's blocks next to each other (they are rotated in place);
  // then those of the key and value heads with 16 consecutive rows next to each other: in a cache in
  // fragment order the same 8 dimensions of 16 consecutive tokens lie together.
  const long q_items = n_tokens * n_heads * blocks;
  for (long idx = blockIdx.x * static_cast<long>(blockDim.x) + threadIdx.x; idx < total; idx += stride) {
    int b, head;
    long token;
    if (idx < q_items) {
      b = static_cast<int>(idx % blocks);
      head = static_cast<int>((idx / blocks) % n_heads);
      token = idx / (static_cast<long>(blocks) * n_heads);
    } else {
      const long j = idx - q_items;
      b = static_cast<int>((j / 16) % blocks);
      head = n_heads + static_cast<int>((j / (16 * blocks)) % (2 * n_kv_heads));
      token = (j / (16L * blocks * 2 * n_kv_heads)) * 16 + j % 16;
      if (token >= n_tokens) continue;
    }
    const bool is_q = head < n_heads, is_v = head >= n_heads + n_kv_heads;
    if (!is_q && !write_kv) continue;
    T* src = qkv + (token * heads_total + head) * head_dim + 16 * b;
    float lo[8], hi[8];
    if constexpr (sizeof(T) == 2) {
      const uint4 l = *reinterpret_cast<const uint4*>(src), h = *reinterpret_cast<const uint4*>(src + 8);
      const uint32_t lw[4] = {l.x, l.y, l.z, l.w}, hw[4] = {h.x, h.y, h.z, h.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[2 * e] = __uint_as_float(lw[e] << 16);
        lo[2 * e + 1] = __uint_as_float(lw[e] & 0xffff0000u);
        hi[2 * e] = __uint_as_float(hw[e] << 16);
        hi[2 * e + 1] = __uint_as_float(hw[e] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        lo[e] = to_float(src[e]);
        hi[e] = to_float(src[8 + e]);
      }
    }
    if (rotate && !is_v) {
      const float2* cs = table + token * (head_dim / 2) + 8 * b;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float2 a = cs[e];
        const float l0 = lo[e], h0 = hi[e];
        lo[e] = l0 * a.x - h0 * a.y;
        hi[e] = h0 * a.x + l0 * a.y;
      }
    }
    if (is_v) {   // values are kept transposed: [page][kv head][dim][token]
      const int slot = slot_map[token];
      const long page = slot / page_tokens, off = slot % page_tokens;
      T* region = v_cache + (page * n_kv_heads + (head - n_heads - n_kv_heads)) * head_dim * page_tokens;
      // dimension 16b + c of the token: 4 elements further for every c in fragment order, a page row otherwise
      T* dst = frag ? region + frag_v_offset(static_cast<int>(off), 16 * b, head_dim) : region + 16L * b * page_tokens + off;
      const long step = frag ? 4 : page_tokens;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        dst[e * step] = from_float<T>(lo[e]);
        dst[(8 + e) * step] = from_float<T>(hi[e]);
      }
      continue;
    }
    T* dst = src;
    long second = 8;   // where the block's second eight elements go, from dst
    if (!is_q) {   // keys: [page][kv head][token][dim], or in fragment order: eight dimensions of 16 tokens together
      const int slot = slot_map[token];
      const long page = slot / page_tokens, off = slot % page_tokens;
      T* region = k_cache + (page * n_kv_heads + (head - n_heads)) * page_tokens * head_dim;
      dst = frag ? region + frag_k_offset(static_cast<int>(off), 16 * b, head_dim) : region + off * head_dim + 16 * b;
      if (frag) second = 16 * 8;
    }
    if constexpr (sizeof(T) == 2) {
      uint32_t lw[4], hw[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lw[e] = static_cast<uint32_t>(bf16_bits_from_float(lo[2 * e])) | (static_cast<uint32_t>(bf16_bits_from_float(lo[2 * e + 1])) << 16);
        hw[e] = static_cast<uint32_t>(bf16_bits_from_float(hi[2 * e])) | (static_cast<uint32_t>(bf16_bits_from_float(hi[2 * e + 1])) << 16);
      }
      *reinterpret_cast<uint4*>(dst) = make_uint4(lw[0], lw[1], lw[2], lw[3]);
      *reinterpret_cast<uint4*>(dst + second) = make_uint4(hw[0], hw[1], hw[2], hw[3]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        dst[e] = from_float<T>(lo[e]);
        dst[second + e] = from_float<T>(hi[e]);
      }
    }
  }
}

// ---- argmax ----------------------------------------------------------------
// Two stages so that a few rows still use many CUs: every block takes one slice of one row and
// writes its best (value, index); one wave per row then picks among the slices.  Equal values
// keep the lower index at every step.
constexpr int kArgmaxSlices = 64;

__device__ inline void better(float& v, int& i, float ov, int oi) {
  if (ov > v || (ov == v && oi < i)) {
    v = ov;
    i = oi;
  }
}

__global__ void argmax_slices_kernel(const float* __restrict__ logits, float* __restrict__ part_v,
                                     int32_t* __restrict__ part_i, int vocab) {
  __shared__ float best_v[kBlock];
  __shared__ int best_i[kBlock];
  const float* row = logits + static_cast<size_t>(blockIdx.x) * vocab;
  const int per = (vocab + kArgmaxSlices - 1) / kArgmaxSlices;
  const int begin = min(vocab, static_cast<int>(blockIdx.y) * per), end = min(vocab, begin + per);
  float v = -FLT_MAX;
  int idx = vocab;  // empty marker: loses every tie against a real index
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) better(v, idx, row[i], i);
  best_v[threadIdx.x] = v;
  best_i[threadIdx.x] = idx;
  __syncthreads();
  for (int h = blockDim.x / 2; h > 0; h >>= 1) {
    if (threadIdx.x < h) better(best_v[threadIdx.x], best_i[threadIdx.x], best_v[threadIdx.x + h], best_i[threadIdx.x + h]);
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    part_v[blockIdx.x * kArgmaxSlices + blockIdx.y] = best_v[0];
    part_i[blockIdx.x * kArgmaxSlices + blockIdx.y] = best_i[0];
  }
}

__global__ void argmax_pick_kernel(const float* __restrict__ part_v, const int32_t* __restrict__ part_i,
                                   int32_t* __restrict__ out, int vocab) {
  float v = part_v[blockIdx.x * kArgmaxSlices + threadIdx.x];
  int idx = part_i[blockIdx.x * kArgmaxSlices + threadIdx.x];
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) better(v, idx, __shfl_xor(v, off, kWave), __shfl_xor(idx, off, kWave));
  if (threadIdx.x == 0) out[blockIdx.x] = idx < vocab ? idx : 0;
}

// ---- temperature sampling --------------------------------------------------
// The law: weights w_i = exp((l_i - max) / T) in float, summed in double; the token is the first i,
// in vocabulary order, at which u * total - (w_0 + ... + w_i) turns negative.  One workgroup a row.
// The vocabulary is cut into groups of 512 consecutive tokens, a lane holding eight in a row (more
// beyond 2,097,152 tokens, so that the groups' sums fit LDS): a lane sums its own tokens in order
// without a word to its neighbours (sums of doubles across lanes go through the LDS crossbar, which
// sixteen waves share), a wave then a group; every pass over the row reads whole cache lines.  The
// groups' sums, a running sum over them (one wave, 64 groups a step) and a last look inside the one
// group where the target is crossed find the token.
// (Sums in another order than the host's one-by-one walk: a boundary may move by one token when u
// falls within rounding of it.)
constexpr int kSampleThreads = 1024;
constexpr int kSampleMaxGroups = 4096;
constexpr int kSamplePerLane = 8;           // consecutive tokens a lane holds of a group
constexpr int kSampleAhead = 4;             // loads of 16 bytes (pairs of them in the second pass) a thread has in flight

__device__ inline double wave_sum_f64(double v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
// inclusive running sum over the wave's lanes, in lane order
__device__ inline double wave_scan_f64(double v, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const double up = __shfl_up(v, off, kWave);
    if (lane >= off) v += up;
  }
  return v;
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(const float* __restrict__ logits,
                                                               const float* __restrict__ temperature,
                                                               const double* __restrict__ u, int32_t* __restrict__ out,
                                                               int vocab) {
  __shared__ double group_sum[kSampleMaxGroups];      // then: the running sum up to and with each group
  constexpr int kWaves = kSampleThreads / kWave;
  __shared__ float best_v[kWaves];
  __shared__ int best_i[kWaves];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const float* row = logits + static_cast<size_t>(blockIdx.x) * vocab;

  // the maximum and where it stands first
  float v = -FLT_MAX;
  int idx = vocab;
  // in fours where every row starts on 16 bytes (the base does and the vocabulary is a multiple of four): no group of
  // four then straddles a row's end
  const bool by_four = vocab % 4 == 0 && reinterpret_cast<uintptr_t>(logits) % 16 == 0;
  if (by_four) {
    const float4* row4 = reinterpret_cast<const float4*>(row);
    const int n4 = vocab / 4;
    for (int at = threadIdx.x; at < n4; at += kSampleAhead * kSampleThreads) {
      float4 t[kSampleAhead];               // the loads first, so that they are in flight together
#pragma unroll
      for (int j = 0; j < kSampleAhead; ++j) {
        const int i4 = at + j * kSampleThreads;
        t[j] = i4 < n4 ? row4[i4] : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int j = 0; j < kSampleAhead; ++j) {
        const int i4 = at + j * kSampleThreads;
        if (i4 < n4) {
          better(v, idx, t[j].x, 4 * i4);
          better(v, idx, t[j].y, 4 * i4 + 1);
          better(v, idx, t[j].z, 4 * i4 + 2);
          better(v, idx, t[j].w, 4 * i4 + 3);
        }
      }
    }
  } else {
    for (int at = threadIdx.x; at < vocab; at += kSampleThreads) better(v, idx, row[at], at);
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) better(v, idx, __shfl_xor(v, off, kWave), __shfl_xor(idx, off, kWave));
  if (lane == 0) {
    best_v[wave] = v;
    best_i[wave] = idx;
  }
  __syncthreads();
  float row_max = best_v[0];
  int best = best_i[0];
  for (int w = 1; w < kWaves; ++w) better(row_max, best, best_v[w], best_i[w]);
  const int arg = best < vocab ? best : 0;
  const float temp = temperature[blockIdx.x];
  if (!(temp > 0.f)) {
    if (threadIdx.x == 0) out[blockIdx.x] = arg;
    return;
  }
  const float inv_t = 1.0f / temp;
  const int per_lane = max(kSamplePerLane, (vocab + kWave * kSampleMaxGroups - 1) / (kWave * kSampleMaxGroups));
  const int group_size = kWave * per_lane;
  const int n_groups = (vocab + group_size - 1) / group_size;
  auto lane_weight_sum = [&](int g) {      // this lane's tokens of group g, in order
    double s = 0.0;
    const int first = g * group_size + lane * per_lane;
    for (int j = 0; j < per_lane; ++j) {
      const int i = first + j;
      if (i < vocab) s += static_cast<double>(expf((row[i] - row_max) * inv_t));
    }
    return s;
  };
  if (by_four && per_lane == kSamplePerLane) {        // a wave's groups at once: their loads are in flight together
    static_assert(kSamplePerLane == 8, "two loads of four a lane");
    for (int g0 = wave; g0 < n_groups; g0 += kWaves * kSampleAhead) {
      float4 t[kSampleAhead][2];
#pragma unroll
      for (int j = 0; j < kSampleAhead; ++j) {
        const int first = (g0 + j * kWaves) * group_size + lane * kSamplePerLane;
#pragma unroll
        for (int h = 0; h < 2; ++h)
          t[j][h] = first + 4 * h < vocab ? *reinterpret_cast<const float4*>(row + first + 4 * h) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int j = 0; j < kSampleAhead; ++j) {
        const int g = g0 + j * kWaves;
        const int first = g * group_size + lane * kSamplePerLane;
        double s = 0.0;                     // the order of lane_weight_sum: the look inside a group sums the same
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          if (first + 4 * h < vocab) {
            s += static_cast<double>(expf((t[j][h].x - row_max) * inv_t));
            s += static_cast<double>(expf((t[j][h].y - row_max) * inv_t));
            s += static_cast<double>(expf((t[j][h].z - row_max) * inv_t));
            s += static_cast<double>(expf((t[j][h].w - row_max) * inv_t));
          }
        }
        s = wave_sum_f64(s);
        if (lane == 0 && g < n_groups) group_sum[g] = s;
      }
    }
  } else {
    for (int g = wave; g < n_groups; g += kWaves) {
      const double s = wave_sum_f64(lane_weight_sum(g));
      if (lane == 0) group_sum[g] = s;
    }
  }
  __syncthreads();
  if (wave != 0) return;

  // one wave: running sums over the groups, 64 at a step; then the first group they cross the target in
  double carry = 0.0;
  for (int c = 0; c < n_groups; c += kWave) {
    const int g = c + lane;
    const double incl = carry + wave_scan_f64(g < n_groups ? group_sum[g] : 0.0, lane);
    if (g < n_groups) group_sum[g] = incl;
    carry = __shfl(incl, kWave - 1, kWave);
  }
  const double target = u[blockIdx.x] * carry;
  int found = n_groups;
  for (int c = 0; c < n_groups && found == n_groups; c += kWave) {
    const int g = c + lane;
    const unsigned long long over = __ballot(g < n_groups && target - group_sum[g] < 0.0);
    if (over != 0ull) found = c + __ffsll(static_cast<long long>(over)) - 1;
  }
  int result = arg;        // rounding may leave the target a hair above zero after the last token
  if (found < n_groups) {
    const double before = found > 0 ? group_sum[found - 1] : 0.0;
    const double mine = lane_weight_sum(found);
    const double upto = before + wave_scan_f64(mine, lane);              // with this lane's tokens
    const unsigned long long over = __ballot(target - upto < 0.0);
    if (over != 0ull) {
      const int at = __ffsll(static_cast<long long>(over)) - 1;          // the lane whose tokens cross it
      double left = target - (upto - mine);
      const int first = found * group_size + lane * per_lane;
      int hit = min(vocab - 1, first + per_lane - 1);
      for (int j = 0; j < per_lane; ++j) {
        const int i = first + j;
        if (i >= vocab) break;
        left -= static_cast<double>(expf((row[i] - row_max) * inv_t));
        if (left < 0.0) {
          hit = i;
          break;
        }
      }
      result = __shfl(hit, at, kWave);
    }
  }
  if (lane == 0) out[blockIdx.x] = result;
}

int grid_for(long total) {
  long g = (total + kBlock - 1) / kBlock;
  if (g < 1) g = 1;
  if (g > 65535L * 16) g = 65535L * 16;
  return static_cast<int>(g);
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_embed_gather(const void* table, int table_dtype, const int32_t* ids, float* out,
                                 int n_tokens, int hidden, int vocab, void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes T=%d H=%d V=%d",
               n_tokens, hidden, vocab);
  if (n_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (table_dtype == kF32) {
    embed_gather_kernel<float><<<n_tokens, kBlock, 0, s>>>(static_cast<const float*>(table), ids, out, hidden);
  } else if (table_dtype == kBF16) {
    embed_gather_kernel<bf16_t><<<n_tokens, kBlock, 0, s>>>(static_cast<const bf16_t*>(table), ids, out, hidden);
  } else {
    return fail("embed_gather: unknown table dtype %d", table_dtype);
  }
  return check_launch("embed_gather");
}

extern "C" int bc4g_rmsnorm(const float* x, const int32_t* rows, const void* w, int w_dtype, void* out,
                            int out_dtype, int n_rows, int hidden, float eps, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && hidden > 0, "rmsnorm: bad sizes rows=%d H=%d", n_rows, hidden);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // widths that are a multiple of 8, up to 8,192: the row stays in registers
  const int chunks = hidden % 8 == 0 ? (hidden + 2047) / 2048 : 0;
#define BC4G_RMS(TW, TO)                                                                                    \
  do {                                                                                                      \
    const TW* wp = static_cast<const TW*>(w);                                                               \
    TO* op = static_cast<TO*>(out);                                                                         \
    if (chunks == 1) rmsnorm_rows_kernel<TW, TO, 1><<<n_rows, 256, 0, s>>>(x, rows, wp, op, hidden, eps);      \
    else if (chunks == 2) rmsnorm_rows_kernel<TW, TO, 2><<<n_rows, 256, 0, s>>>(x, rows, wp, op, hidden, eps); \
    else if (chunks == 3 || chunks == 4)                                                                    \
      rmsnorm_rows_kernel<TW, TO, 4><<<n_rows, 256, 0, s>>>(x, rows, wp, op, hidden, eps);                   \
    else rmsnorm_kernel<TW, TO><<<n_rows, kBlock, 0, s>>>(x, rows, wp, op, hidden, eps);                     \
  } while (0)
  if (w_dtype == kF32 && out_dtype == kF32) BC4G_RMS(float, float);
  else if (w_dtype == kF32 && out_dtype == kBF16) BC4G_RMS(float, bf16_t);
  else if (w_dtype == kBF16 && out_dtype == kF32) BC4G_RMS(bf16_t, float);
  else if (w_dtype == kBF16 && out_dtype == kBF16) BC4G_RMS(bf16_t, bf16_t);
  else return fail("rmsnorm: unknown dtypes w=%d out=%d", w_dtype, out_dtype);
#undef BC4G_RMS
  return check_launch("rmsnorm");
}

extern "C" int bc4g_rmsnorm_sum(float* x, const float* parts, int n_parts, const void* w, int w_dtype, void* out,
                                int out_dtype, int n_rows, int hidden, float eps, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && hidden > 0 && hidden % 8 == 0 && hidden <= 8192 && n_parts >= 1 && n_parts <= 16,
               "rmsnorm_sum: rows=%d of H=%d (a multiple of 8, at most 8192) in %d parts (1 to 16)", n_rows, hidden, n_parts);
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int chunks = (hidden + 2047) / 2048;
#define BC4G_RMS_SUM(TW, TO)                                                                                              \
  do {                                                                                                                    \
    const TW* wp = static_cast<const TW*>(w);                                                                             \
    TO* op = static_cast<TO*>(out);                                                                                       \
    if (chunks == 1) rmsnorm_sum_rows_kernel<TW, TO, 1><<<n_rows, 256, 0, s>>>(x, parts, n_parts, wp, op, n_rows, hidden, eps);      \
    else if (chunks == 2) rmsnorm_sum_rows_kernel<TW, TO, 2><<<n_rows, 256, 0, s>>>(x, parts, n_parts, wp, op, n_rows, hidden, eps); \
    else rmsnorm_sum_rows_kernel<TW, TO, 4><<<n_rows, 256, 0, s>>>(x, parts, n_parts, wp, op, n_rows, hidden, eps);                  \
  } while (0)
  if (w_dtype == kF32 && out_dtype == kBF16) BC4G_RMS_SUM(float, bf16_t);
  else if (w_dtype == kBF16 && out_dtype == kBF16) BC4G_RMS_SUM(bf16_t, bf16_t);
  else return fail("rmsnorm_sum: unknown dtypes w=%d out=%d (the output is bfloat16)", w_dtype, out_dtype);
#undef BC4G_RMS_SUM
  return check_launch("rmsnorm_sum");
}

extern "C" int bc4g_swiglu(const void* gu, void* out, int dtype, int n_tokens, int inter, int interleaved,
                           void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && inter > 0, "swiglu: bad sizes T=%d I=%d", n_tokens, inter);
  BC4G_REQUIRE(!interleaved || inter % 8 == 0, "swiglu: the interleaved layout needs I=%d to be a multiple of 8", inter);
  if (n_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_tokens) * inter;
  if (dtype == kF32) {
    swiglu_kernel<float><<<grid_for(total), kBlock, 0, s>>>(static_cast<const float*>(gu),
                                                            static_cast<float*>(out), total, inter, interleaved);
  } else if (dtype == kBF16) {
    swiglu_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(static_cast<const bf16_t*>(gu),
                                                             static_cast<bf16_t*>(out), total, inter, interleaved);
  } else {
    return fail("swiglu: unknown dtype %d", dtype);
  }
  return check_launch("swiglu");
}

extern "C" int bc4g_rope_kv_write(void* qkv, int dtype, const int32_t* positions, const int32_t* slot_map,
                                  void* k_cache, void* v_cache, int n_tokens, int n_heads, int n_kv_heads,
                                  int head_dim, int rotary_dim, float theta, int page_tokens, int num_pages,
                                  int write_kv, int block_pairs, void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0, "rope_kv_write: bad sizes T=%d heads=%d/%d",
               n_tokens, n_heads, n_kv_heads);
  BC4G_REQUIRE(head_dim > 0 && head_dim % 2 == 0, "rope_kv_write: head_dim %d must be even", head_dim);
  BC4G_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
               "rope_kv_write: rotary_dim %d must be even and at most head_dim %d", rotary_dim, head_dim);
  BC4G_REQUIRE(!write_kv || (page_tokens > 0 && num_pages > 0 && k_cache && v_cache && slot_map),
               "rope_kv_write: cache write asked for without a cache");
  BC4G_REQUIRE(rotary_dim == 0 || (positions && theta > 0.f), "rope_kv_write: rotation needs positions and theta > 0");
  BC4G_REQUIRE(!block_pairs || (head_dim % 16 == 0 && (rotary_dim == 0 || rotary_dim == head_dim)),
               "rope_kv_write: the block layout needs head_dim %d to be a multiple of 16 and a full rotation", head_dim);
  if (n_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const long total = static_cast<long>(n_tokens) * (n_heads + 2 * n_kv_heads) * (head_dim / 2);
  if (dtype == kF32) {
    rope_kv_write_kernel<float><<<grid_for(total), kBlock, 0, s>>>(
        static_cast<float*>(qkv), positions, slot_map, static_cast<float*>(k_cache),
        static_cast<float*>(v_cache), total, n_heads, n_kv_heads, head_dim, rotary_dim, theta, page_tokens, write_kv,
        block_pairs, 0);
  } else if (dtype == kBF16) {
    rope_kv_write_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(
        static_cast<bf16_t*>(qkv), positions, slot_map, static_cast<bf16_t*>(k_cache),
        static_cast<bf16_t*>(v_cache), total, n_heads, n_kv_heads, head_dim, rotary_dim, theta, page_tokens, write_kv,
        block_pairs, cache_fragment_order(true, head_dim, page_tokens) ? 1 : 0);
  } else {
    return fail("rope_kv_write: unknown dtype %d", dtype);
  }
  return check_launch("rope_kv_write");
}

extern "C" int bc4g_rope_table(const int32_t* positions, float* table, int n_tokens, int rotary_dim, float theta,
                               void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && rotary_dim > 0 && rotary_dim % 2 == 0 && theta > 0.f && positions && table,
               "rope_table: bad arguments (T=%d, rotary_dim=%d)", n_tokens, rotary_dim);
  if (n_tokens == 0) return 0;
  const long total = static_cast<long>(n_tokens) * (rotary_dim / 2);
  rope_table_kernel<<<grid_for(total), kBlock, 0, static_cast<hipStream_t>(stream)>>>(
      positions, reinterpret_cast<float2*>(table), total, rotary_dim / 2, theta);
  return check_launch("rope_table");
}

extern "C" int bc4g_rope_kv_write_blocks(void* qkv, int dtype, const float* table, const int32_t* slot_map,
                                         void* k_cache, void* v_cache, int n_tokens, int n_heads, int n_kv_heads,
                                         int head_dim, int rotate, int page_tokens, int write_kv, void* stream) {
  BC4G_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0, "rope_kv_write_blocks: bad sizes T=%d heads=%d/%d",
               n_tokens, n_heads, n_kv_heads);
  BC4G_REQUIRE(head_dim > 0 && head_dim % 16 == 0, "rope_kv_write_blocks: head_dim %d must be a multiple of 16", head_dim);
  BC4G_REQUIRE(!write_kv || (page_tokens > 0 && k_cache && v_cache && slot_map),
               "rope_kv_write_blocks: cache write asked for without a cache");
  BC4G_REQUIRE(!rotate || table, "rope_kv_write_blocks: rotation needs the table of angles");
  if (n_tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // (the key and value heads' items are counted for whole groups of 16 rows)
  const long total = (static_cast<long>(n_tokens) * n_heads + ((n_tokens + 15) / 16) * 16L * 2 * n_kv_heads) * (head_dim / 16);
  const float2* tab = reinterpret_cast<const float2*>(table);
  if (dtype == kF32) {
    rope_kv_write_blocks_kernel<float><<<grid_for(total), kBlock, 0, s>>>(
        static_cast<float*>(qkv), tab, slot_map, static_cast<float*>(k_cache), static_cast<float*>(v_cache), total,
        n_tokens, n_heads, n_kv_heads, head_dim, rotate, page_tokens, write_kv, 0);
  } else if (dtype == kBF16) {
    rope_kv_write_blocks_kernel<bf16_t><<<grid_for(total), kBlock, 0, s>>>(
        static_cast<bf16_t*>(qkv), tab, slot_map, static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), total,
        n_tokens, n_heads, n_kv_heads, head_dim, rotate, page_tokens, write_kv,
        cache_fragment_order(true, head_dim, page_tokens) ? 1 : 0);
  } else {
    return fail("rope_kv_write_blocks: unknown dtype %d", dtype);
  }
  return check_launch("rope_kv_write_blocks");
}

extern "C" int bc4g_argmax(const float* logits, int32_t* out, float* part_v, int32_t* part_i, int n_rows, int vocab,
                           void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && vocab > 0 && n_rows <= 65535, "argmax: bad sizes rows=%d V=%d", n_rows, vocab);
  BC4G_REQUIRE(part_v && part_i, "argmax: the slice buffers ([rows, 64] each) are missing");
  if (n_rows == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  static_assert(kArgmaxSlices == kWave, "one lane per slice in the second stage");
  argmax_slices_kernel<<<dim3(n_rows, kArgmaxSlices), kBlock, 0, s>>>(logits, part_v, part_i, vocab);
  if (int e = check_launch("argmax_slices")) return e;
  argmax_pick_kernel<<<n_rows, kWave, 0, s>>>(part_v, part_i, out, vocab);
  return check_launch("argmax_pick");
}

// ---- argmax for callers that cannot allocate ------------------------------------------------
// The two stages of bc4g_argmax hand the slices' bests over through device memory that the caller
// brings as a workspace.  Here that memory is an array of the library's own: every GPU the library
// runs on holds a copy of it (512 KiB) at an address of its own until the process ends, and all calls
// on a GPU share it.  In host code the array's name is a stand-in, not a device address: the address
// is asked for once per device (hipGetSymbolAddress, with that device current) and kept, and only
// that pointer is ever handed to a kernel.
constexpr int kArgmaxStaticMaxRows = 1024;
constexpr size_t kArgmaxStaticValueBytes = static_cast<size_t>(kArgmaxStaticMaxRows) * kArgmaxSlices * sizeof(float);
constexpr size_t kArgmaxStaticBytes = kArgmaxStaticValueBytes + static_cast<size_t>(kArgmaxStaticMaxRows) * kArgmaxSlices * sizeof(int32_t);
static __device__ __align__(256) unsigned char scratch[kArgmaxStaticBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {nullptr};

// The address of `scratch` on the current device (asked for at the first call on that device).
int scratch_on_current_device(unsigned char** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail("argmax_static: no current device: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail("argmax_static: device %d is beyond the %d this library keeps track of", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail("argmax_static: cannot find the scratch array on device %d: %s", dev, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *ptr = static_cast<unsigned char*>(g_scratch_ptr[dev]);
  return 0;
}
}  // namespace

extern "C" int bc4g_argmax_static_max_rows() { return kArgmaxStaticMaxRows; }

extern "C" int bc4g_argmax_static(const float* logits, int32_t* out, int n_rows, int vocab, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && vocab > 0, "argmax_static: bad sizes rows=%d V=%d", n_rows, vocab);
  BC4G_REQUIRE(n_rows <= kArgmaxStaticMaxRows, "argmax_static: %d rows are more than the %d the library's own scratch memory holds; "
               "use bc4g_argmax with a workspace of the caller's", n_rows, kArgmaxStaticMaxRows);
  BC4G_REQUIRE(logits && out, "argmax_static: logits and out are needed");
  if (n_rows == 0) return 0;
  unsigned char* base = nullptr;
  if (int e = scratch_on_current_device(&base)) return e;
  // nothing in the array has to start at zero: the first stage writes every slot the second reads
  float* part_v = reinterpret_cast<float*>(base);
  int32_t* part_i = reinterpret_cast<int32_t*>(base + kArgmaxStaticValueBytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  argmax_slices_kernel<<<dim3(n_rows, kArgmaxSlices), kBlock, 0, s>>>(logits, part_v, part_i, vocab);
  if (int e = check_launch("argmax_slices")) return e;
  argmax_pick_kernel<<<n_rows, kWave, 0, s>>>(part_v, part_i, out, vocab);
  return check_launch("argmax_pick");
}

extern "C" int bc4g_sample(const float* logits, const float* temperature, const double* u, int32_t* out,
                           int n_rows, int vocab, void* stream) {
  BC4G_REQUIRE(n_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d V=%d", n_rows, vocab);
  if (n_rows == 0) return 0;
  sample_kernel<<<n_rows, kSampleThreads, 0, static_cast<hipStream_t>(stream)>>>(logits, temperature, u, out, vocab);
  return check_launch("sample");
}
