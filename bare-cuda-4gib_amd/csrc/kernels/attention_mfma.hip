// Causal softmax attention over the paged cache on the matrix cores, bfloat16, for prompt
// portions and decoded tokens alike.
//
// One wave owns a tile of 16 query rows: `tpt` consecutive tokens of one request times `hg`
// query heads that share one key/value head (hg * tpt <= 16).  It walks the keys it may see in
// tiles of 32 and never writes scores to memory:
//   S^T = K Q^T   16x16x32 MFMAs with the keys as rows, so that a lane holds one query row's
//                 scores and the softmax statistics are reductions inside a lane plus two
//                 shuffles;  K rows come straight from the cache pages as the A operand
//   online softmax in float, base 2, masked by absolute position (and the window)
//   O^T += V^T P^T   with P^T taken from the score registers as the B operand and V^T loaded
//                 from the transposed value pages (8-byte loads of 4 consecutive tokens)
// With n_splits > 1 the key range is cut into that many parts (grid z); each part writes
// unnormalized float partials, and attention_merge_kernel combines them.
//
// A row reads keys max(0, p - window + 1) .. p only.  Keys beyond the tile's last position may
// never have been written: their scores are replaced by -inf and their values by zero, so that
// whatever lies in those places (NaN included) cannot reach the sums.
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr float kLog2e = 1.4426950408889634f;

struct AttnArgs {
  const bf16_t* qkv;
  bf16_t* out;                 // [T, n_heads * d]               (n_splits == 1)
  float* part_o;               // [n_splits, T, n_heads, d]      (n_splits > 1), unnormalized
  float* part_ml;              // [n_splits, T, n_heads, 2]      running max (base 2) and sum
  const bf16_t* k_cache;       // [pages, n_kv, P, d]
  const bf16_t* v_cache;       // [pages, n_kv, d, P]
  const int32_t* block_table;  // [S, table_stride]
  const int32_t* seq_start;    // [S + 1] first row of each request in the batch
  const int32_t* seq_ctx;      // [S] tokens cached before this step
  const int32_t* tile_start;   // [S + 1] first tile of each request
  int table_stride, n_seqs, n_tiles, n_tokens;
  int n_heads, n_kv_heads, head_dim, page_tokens, window;
  int hg, tpt, n_sub;          // heads per tile, tokens per tile, head sub-groups per kv head
  int n_splits;
  float scale_log2;            // softmax scale times log2(e)
};

// DJ: k-steps of 32 over head_dim for the scores; DB: blocks of 16 output dimensions.
template <int DJ, int DB>
__global__ __launch_bounds__(kWavesPerBlock * kWave) void attention_mfma_kernel(const AttnArgs a) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int col = lane % 16, grp = lane / 16;
  const int tile = blockIdx.x * kWavesPerBlock + wave;
  if (tile >= a.n_tiles) return;   // no block-wide barrier below: waves are independent

  // which request this tile belongs to
  int lo_s = 0, hi_s = a.n_seqs - 1;
  while (lo_s < hi_s) {
    const int mid = (lo_s + hi_s + 1) >> 1;
    if (a.tile_start[mid] <= tile) lo_s = mid; else hi_s = mid - 1;
  }
  const int s = lo_s;
  const int row0 = a.seq_start[s];
  const int q_len = a.seq_start[s + 1] - row0;
  const int ctx = a.seq_ctx[s];
  const int tok0 = (tile - a.tile_start[s]) * a.tpt;
  const int ntok = min(a.tpt, q_len - tok0);
  const int kvh = blockIdx.y / a.n_sub, hsub = blockIdx.y % a.n_sub;
  const int group = a.n_heads / a.n_kv_heads;
  const int d = a.head_dim, P = a.page_tokens;
  const int32_t* table = a.block_table + static_cast<long>(s) * a.table_stride;

  // this lane's query row (as B operand and as owner of one row's statistics)
  const int q_tok = col / a.hg, q_hsub = col % a.hg;
  const int q_head_in_group = hsub * a.hg + q_hsub;
  const bool q_ok = q_tok < ntok && q_head_in_group < group;
  const int q_head = kvh * group + q_head_in_group;
  const int q_pos = ctx + tok0 + q_tok;
  const int q_lo = (a.window > 0 && q_pos - a.window + 1 > 0) ? q_pos - a.window + 1 : 0;
  const long qkv_stride = static_cast<long>(a.n_heads + 2 * a.n_kv_heads) * d;

  uint4 qf[DJ];
#pragma unroll
  for (int j = 0; j < DJ; ++j) {
    const int c = 32 * j + 8 * grp;
    qf[j] = (q_ok && c < d) ? load16(a.qkv + (row0 + tok0 + q_tok) * qkv_stride + static_cast<long>(q_head) * d + c)
                            : zero16();
  }

  const int pos_min = ctx + tok0, pos_max = ctx + tok0 + ntok - 1;
  const int lo_min = (a.window > 0 && pos_min - a.window + 1 > 0) ? pos_min - a.window + 1 : 0;
  const int kt_first = lo_min / 32, kt_last = pos_max / 32;
  const int n_kt = kt_last - kt_first + 1;
  const int per_split = (n_kt + a.n_splits - 1) / a.n_splits;
  const int kt_begin = kt_first + blockIdx.z * per_split;
  const int kt_end = min(kt_last + 1, kt_begin + per_split);

  float m_run = -INFINITY, l_run = 0.f;
  floatx4 o[DB];
#pragma unroll
  for (int b = 0; b < DB; ++b) o[b] = floatx4{0.f, 0.f, 0.f, 0.f};

  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const int key0 = kt * 32;
    floatx4 sc[2];
    long vbase[2];
    bool sub_ok[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kb = key0 + 16 * h;
      sub_ok[h] = kb <= pos_max && kb + 15 >= lo_min;
      sc[h] = floatx4{0.f, 0.f, 0.f, 0.f};
      vbase[h] = 0;
      if (sub_ok[h]) {
        const long page = table[kb / P];
        const int off = kb % P;
        const bf16_t* kptr = a.k_cache + ((page * a.n_kv_heads + kvh) * P + off + col) * d + 8 * grp;
        vbase[h] = (page * a.n_kv_heads + kvh) * static_cast<long>(d) * P + off + 4 * grp;
#pragma unroll
        for (int j = 0; j < DJ; ++j) {
          const uint4 kf = (32 * j + 8 * grp < d) ? load16(kptr + 32 * j) : zero16();
          sc[h] = mfma_16x16x32(kf, qf[j], sc[h]);
        }
      }
    }
    // mask by position; this lane holds, for its query row, keys key0 + 16h + 4*grp + r
    float sv[8];
    float m_tile = -INFINITY;
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = key0 + 16 * h + 4 * grp + r;
        const bool vis = sub_ok[h] && q_ok && key <= q_pos && key >= q_lo;
        const float v = vis ? sc[h][r] * a.scale_log2 : -INFINITY;
        sv[4 * h + r] = v;
        m_tile = fmaxf(m_tile, v);
      }
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, kWave));
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, kWave));
    const float m_new = fmaxf(m_run, m_tile);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = exp2f(m_run - m_safe);   // 0 while nothing has been seen
    float psum = 0.f;
    uint32_t pk[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float p0 = exp2f(sv[2 * i] - m_safe), p1 = exp2f(sv[2 * i + 1] - m_safe);
      psum += p0 + p1;
      pk[i] = static_cast<uint32_t>(bf16_bits_from_float(p0)) |
              (static_cast<uint32_t>(bf16_bits_from_float(p1)) << 16);
    }
    l_run = l_run * alpha + psum;
    m_run = m_new;
    const uint4 pf = make_uint4(pk[0], pk[1], pk[2], pk[3]);

    // values of keys past the tile's last position are replaced by zero
    uint32_t vmask[4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kb = key0 + 16 * h + 4 * grp;
      vmask[2 * h] = (kb <= pos_max ? 0xffffu : 0u) | (kb + 1 <= pos_max ? 0xffff0000u : 0u);
      vmask[2 * h + 1] = (kb + 2 <= pos_max ? 0xffffu : 0u) | (kb + 3 <= pos_max ? 0xffff0000u : 0u);
    }
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      if (16 * b >= d) break;   // DB is the most blocks this instantiation holds
      uint2 v0 = make_uint2(0u, 0u), v1 = make_uint2(0u, 0u);
      const long dim_off = static_cast<long>(16 * b + col) * P;
      if (sub_ok[0]) v0 = *reinterpret_cast<const uint2*>(a.v_cache + vbase[0] + dim_off);
      if (sub_ok[1]) v1 = *reinterpret_cast<const uint2*>(a.v_cache + vbase[1] + dim_off);
      const uint4 vf = make_uint4(v0.x & vmask[0], v0.y & vmask[1], v1.x & vmask[2], v1.y & vmask[3]);
#pragma unroll
      for (int r = 0; r < 4; ++r) o[b][r] *= alpha;
      o[b] = mfma_16x16x32(vf, pf, o[b]);
    }
  }

  float l_tot = l_run + __shfl_xor(l_run, 16, kWave);
  l_tot += __shfl_xor(l_tot, 32, kWave);
  if (!q_ok) return;
  const long row = row0 + tok0 + q_tok;
  if (a.n_splits == 1) {
    const float inv = 1.0f / l_tot;
    bf16_t* dst = a.out + (row * a.n_heads + q_head) * d + 4 * grp;
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      if (16 * b >= d) break;
      uint2 pack;
      pack.x = static_cast<uint32_t>(bf16_bits_from_float(o[b][0] * inv)) |
               (static_cast<uint32_t>(bf16_bits_from_float(o[b][1] * inv)) << 16);
      pack.y = static_cast<uint32_t>(bf16_bits_from_float(o[b][2] * inv)) |
               (static_cast<uint32_t>(bf16_bits_from_float(o[b][3] * inv)) << 16);
      *reinterpret_cast<uint2*>(dst + 16 * b) = pack;
    }
  } else {
    const long slot = (static_cast<long>(blockIdx.z) * a.n_tokens + row) * a.n_heads + q_head;
    float* dst = a.part_o + slot * d + 4 * grp;
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      if (16 * b >= d) break;
      *reinterpret_cast<floatx4*>(dst + 16 * b) = o[b];
    }
    if (grp == 0) {
      a.part_ml[slot * 2] = m_run;
      a.part_ml[slot * 2 + 1] = l_tot;
    }
  }
}

// out[row, head, :] = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, parts added in order of z.
// One wave per (row, head), up to 64 parts: lane z reads part z's statistics, the weights go
// through LDS, and every lane then sums its output dimensions over the parts.
constexpr int kMaxSplits = 64;

__global__ __launch_bounds__(kWave) void attention_merge_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                bf16_t* __restrict__ out, int n_splits,
                                                                long n_rows_heads, int d) {
  __shared__ float weight[kMaxSplits];
  const long rh = blockIdx.x;
  const int lane = threadIdx.x;
  float mz = -INFINITY, lz = 0.f;
  if (lane < n_splits) {
    const float2 ml = *reinterpret_cast<const float2*>(part_ml + (lane * n_rows_heads + rh) * 2);
    mz = ml.x;
    lz = ml.y;
  }
  const float m = wave_max(mz);
  const float wz = (mz == -INFINITY) ? 0.f : exp2f(mz - m);
  weight[lane] = wz;
  // the sum over parts in order of z, the same in every lane
  __syncthreads();
  float l = 0.f;
  for (int z = 0; z < n_splits; ++z) l += weight[z] * __shfl(lz, z, kWave);
  const float inv = 1.0f / l;
  for (int c = lane; c < d; c += kWave) {
    float acc = 0.f;
#pragma unroll 8
    for (int z = 0; z < n_splits; ++z) acc += weight[z] * part_o[(z * n_rows_heads + rh) * d + c];
    out[rh * d + c] = from_float<bf16_t>(acc * inv);
  }
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_attention_mfma(const void* qkv, void* out, float* part_o, float* part_ml, const void* k_cache,
                                   const void* v_cache, const int32_t* block_table, int table_stride,
                                   const int32_t* seq_start, const int32_t* seq_ctx, const int32_t* tile_start,
                                   int n_seqs, int n_tiles, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                   int page_tokens, int window, float scale, int tokens_per_tile, int n_splits,
                                   void* stream) {
  BC4G_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "attention_mfma: bad heads %d/%d",
               n_heads, n_kv_heads);
  BC4G_REQUIRE(head_dim >= 16 && head_dim <= 256 && head_dim % 16 == 0,
               "attention_mfma: head_dim %d must be a multiple of 16 up to 256", head_dim);
  BC4G_REQUIRE(page_tokens > 0 && page_tokens % 16 == 0, "attention_mfma: page_tokens %d must be a multiple of 16",
               page_tokens);
  BC4G_REQUIRE(n_splits >= 1 && n_splits <= kMaxSplits && (n_splits == 1 || (part_o && part_ml)),
               "attention_mfma: the split count %d must lie in 1..64", n_splits);
  BC4G_REQUIRE(window >= 0 && table_stride > 0 && n_seqs > 0, "attention_mfma: bad sizes");
  if (n_tiles == 0 || n_tokens == 0) return 0;
  const int group = n_heads / n_kv_heads;
  AttnArgs a;
  a.qkv = static_cast<const bf16_t*>(qkv);
  a.out = static_cast<bf16_t*>(out);
  a.part_o = part_o;
  a.part_ml = part_ml;
  a.k_cache = static_cast<const bf16_t*>(k_cache);
  a.v_cache = static_cast<const bf16_t*>(v_cache);
  a.block_table = block_table;
  a.seq_start = seq_start;
  a.seq_ctx = seq_ctx;
  a.tile_start = tile_start;
  a.table_stride = table_stride;
  a.n_seqs = n_seqs;
  a.n_tiles = n_tiles;
  a.n_tokens = n_tokens;
  a.n_heads = n_heads;
  a.n_kv_heads = n_kv_heads;
  a.head_dim = head_dim;
  a.page_tokens = page_tokens;
  a.window = window;
  a.hg = group < 16 ? group : 16;
  a.tpt = tokens_per_tile;
  a.n_sub = (group + a.hg - 1) / a.hg;
  a.n_splits = n_splits;
  a.scale_log2 = scale * kLog2e;
  BC4G_REQUIRE(a.tpt >= 1 && a.tpt * a.hg <= 16, "attention_mfma: %d tokens x %d heads do not fit a 16-row tile",
               a.tpt, a.hg);
  BC4G_REQUIRE(n_kv_heads * a.n_sub <= 65535, "attention_mfma: too many heads for the grid");
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid((n_tiles + kWavesPerBlock - 1) / kWavesPerBlock, n_kv_heads * a.n_sub, n_splits);
  dim3 block(kWavesPerBlock * kWave);
  const int dj = (head_dim + 31) / 32, db = head_dim / 16;
  if (dj <= 2 && db <= 4) attention_mfma_kernel<2, 4><<<grid, block, 0, s>>>(a);
  else if (dj <= 4 && db <= 8) attention_mfma_kernel<4, 8><<<grid, block, 0, s>>>(a);
  else attention_mfma_kernel<8, 16><<<grid, block, 0, s>>>(a);
  if (int e = check_launch("attention_mfma")) return e;
  if (n_splits > 1) {
    const long rows_heads = static_cast<long>(n_tokens) * n_heads;
    BC4G_REQUIRE(rows_heads <= 2147483647L, "attention_mfma: too many rows to merge");
    attention_merge_kernel<<<static_cast<unsigned>(rows_heads), 64, 0, s>>>(part_o, part_ml, a.out, n_splits,
                                                                             rows_heads, head_dim);
    return check_launch("attention_merge");
  }
  return 0;
}
