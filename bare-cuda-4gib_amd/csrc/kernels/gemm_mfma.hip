// out[m, n] (+)= sum_k a[m, k] * w[n, k], bfloat16 operands, float accumulation on the matrix
// cores: the product of prompt portions (many rows).
//
// Both operands are contiguous in k.  A workgroup computes a tile of the output in k-steps of 64:
// the rows of a and of w that the tile needs are staged in LDS, every wave reads its fragments there
// and feeds 32x32x16 MFMAs.  Two forms:
//  - gemm_mfma_direct_kernel: the operand tiles go from memory into LDS without passing registers
//    (k a multiple of 64, operands on 16-byte boundaries).  Tiles of 256 x 256, 256 x 192,
//    256 x 128, 128 x 128 or 64 x 64 (and 128 x 64 for q|k|v), whichever lets the busiest CU finish first.
//  - gemm_mfma_staged_kernel: through registers, 128 x 128 tiles; any k that is a multiple of 8.
// Every output element is accumulated over k in ascending order in both, whatever the number of
// rows and the tile: the same bits whichever form and tile a shape selects.
// Rows and columns beyond the matrix are not stored.
//
// What bounds these kernels (clock reads per workgroup, hardware counters): the loop over k is 85-90 %
// of a tile's time, with the matrix cores busy 40-50 % of it -- a step's loads, fragment reads and
// MFMAs overlap only so far between two barriers, although LDS (no bank conflicts, a third of its
// cycles in use) and memory (a ring of three stages is no faster than one of two) both have room;
// a tile of 128 x 64 was bound by what all CUs pull from L2 together (19 TB/s); the rest
// is the stores after the loop, which all CUs issue at the same time.  More waves a CU (this form
// spends no registers on staging) and larger tiles (less traffic per FLOP) are what helped.
//
// Workgroups are numbered so that those sharing rows of a and of w run on the same XCD at the same
// time (tile_of).
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLdsStride = kBK + 8;   // elements; 144 bytes
constexpr int kXcds = 8;

// kSwigluBf16: every 16 rows of w are eight gate rows and the eight up rows of the same outputs;
// out [m, n / 2] = silu(gate) * up.  A gate and its up lie eight columns apart in the product.
// kRopeKvBf16: w holds query, key and value heads with every head's rows in blocks of 16 (eight dimensions, then their
// rotation partners, which so lie eight columns apart in the product): queries are stored rotated, keys go rotated
// into their pages, values into theirs (operands straight into LDS only).
// kSwigluScaledBf16: the same for rows of a that lack their RMSNorm's common factor (a = bfloat16(residual * g), as the
// product that last added to the residual left it, with every row's sum of squares in parts): a row's sums are
// multiplied by 1 / sqrt(sum of squares / k + eps) before the activation (operands straight into LDS only).
enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAccumF32 = 2, kSwigluBf16 = 3, kRopeKvBf16 = 4, kSwigluScaledBf16 = 5 };

constexpr int kPartSums = 8;  // chains a row's parts are added in: chain j takes parts j, j + 8, ... in ascending order, and the
                              // chains are added in order of j -- the order of the weight-streaming kernel, so the same factor
struct RowScaleArgs {
  const float* parts;         // [blocks][stride]: block b's share of every row's sum of squares
  int blocks, stride;
  float eps;
};
// a patch's rows' sums in LDS ([kPartSums][stride], from the patch's first row on) and what finishes them
struct RowScale {
  const float* sums = nullptr;
  int stride = 0;
  float inv_k = 0.f, eps = 0.f;
};

struct RopeKvArgs {
  const float2* table;        // [m, head_dim / 2] (cos, sin) of every row's position and pair (null: no rotation)
  const int32_t* slot_map;    // [m] page * page_tokens + offset
  bf16_t* k_cache;            // [pages, n_kv, page_tokens, d], or every [page_tokens, d] in fragment order
  bf16_t* v_cache;            // [pages, n_kv, d, page_tokens], or likewise
  int n_heads, n_kv_heads, head_dim, page_tokens, write_kv;
  int fragment_order;         // how the cache's pages are laid out (cache_fragment_order)
};

// Which tile a workgroup takes.  Workgroups are dealt to the 8 XCDs in turn, each with an L2 of its
// own: consecutive logical ids stay on one XCD and walk the output in bands of kBand rows of tiles,
// m fastest inside a band -- so the 32 tiles an XCD works on at one time are 8 x 4 of them, which
// share their rows of a and of w in that L2 (with all of m fastest, 8,192 rows were 32 tiles of one
// column, each with rows of a of its own: measured 807 -> 896 TFLOP/s for 8192 x 28672 x 4096).
constexpr int kBand = 8;
__device__ inline void tile_of(int block, int m_blocks, int n_blocks, int& bm, int& bn) {
  const int total = m_blocks * n_blocks;
  int logical = block;
  if (total % kXcds == 0) logical = (block % kXcds) * (total / kXcds) + block / kXcds;
  const int per_band = kBand * n_blocks;
  const int first = (logical / per_band) * kBand;
  const int rows = min(kBand, m_blocks - first);
  const int in_band = logical % per_band;
  bm = first + in_band % rows;
  bn = in_band / rows;
}

// Stores ROWS x COLS floats (stride COLS + 4) from LDS with the epilogue, THREADS threads together.
template <int EPI, int THREADS, int ROWS, int COLS>
__device__ inline void store_patch(const float* patch, void* __restrict__ out, int m, int n, long m0, long n0, int tid,
                                   const RowScale& rs = RowScale{}) {
  constexpr int kStride = COLS + 4;
  if constexpr (EPI == kSwigluBf16 || EPI == kSwigluScaledBf16) {
    // (a block of 16 columns -- eight gates, then their eight ups -- a thread: eight outputs, stored at once)
    const long n_out = n / 2;
    for (int c = tid; c < ROWS * (COLS / 16); c += THREADS) {
      const int row = c / (COLS / 16), col = (c % (COLS / 16)) * 16;
      const long gm = m0 + row, gn = n0 + col;
      if (gm >= m || gn >= n) continue;
      const float* src = patch + row * kStride + col;
      const floatx4 g0 = *reinterpret_cast<const floatx4*>(src), g1 = *reinterpret_cast<const floatx4*>(src + 4);
      const floatx4 u0 = *reinterpret_cast<const floatx4*>(src + 8), u1 = *reinterpret_cast<const floatx4*>(src + 12);
      float scale = 1.f;
      if constexpr (EPI == kSwigluScaledBf16) {
        float ssq = 0.f;
#pragma unroll
        for (int j = 0; j < kPartSums; ++j) ssq += rs.sums[j * rs.stride + row];
        scale = 1.0f / sqrtf(ssq * rs.inv_k + rs.eps);
      }
      float v[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = silu_quick(g0[e] * scale) * (u0[e] * scale);
        v[4 + e] = silu_quick(g1[e] * scale) * (u1[e] * scale);
      }
      bf16_t* dst = static_cast<bf16_t*>(out) + gm * n_out + (gn / 16) * 8;
      if (n_out % 8 == 0) {
        uint4 pk;
        pk.x = static_cast<uint32_t>(bf16_bits_from_float(v[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
        pk.y = static_cast<uint32_t>(bf16_bits_from_float(v[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
        pk.z = static_cast<uint32_t>(bf16_bits_from_float(v[4])) | (static_cast<uint32_t>(bf16_bits_from_float(v[5])) << 16);
        pk.w = static_cast<uint32_t>(bf16_bits_from_float(v[6])) | (static_cast<uint32_t>(bf16_bits_from_float(v[7])) << 16);
        *reinterpret_cast<uint4*>(dst) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) dst[e] = from_float<bf16_t>(v[e]);
      }
    }
  } else if (EPI == kStoreBf16 && n % 8 == 0) {
    // (eight columns a thread, stored at once: 16-byte stores where 8-byte ones were, 108 -> 102 us for a wide product)
    for (int c = tid; c < ROWS * (COLS / 8); c += THREADS) {
      const int row = c / (COLS / 8), col = (c % (COLS / 8)) * 8;
      const long gm = m0 + row, gn = n0 + col;
      if (gm >= m || gn >= n) continue;
      const floatx4 v0 = *reinterpret_cast<const floatx4*>(patch + row * kStride + col);
      const floatx4 v1 = *reinterpret_cast<const floatx4*>(patch + row * kStride + col + 4);
      uint4 pk;
      pk.x = static_cast<uint32_t>(bf16_bits_from_float(v0[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v0[1])) << 16);
      pk.y = static_cast<uint32_t>(bf16_bits_from_float(v0[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v0[3])) << 16);
      pk.z = static_cast<uint32_t>(bf16_bits_from_float(v1[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v1[1])) << 16);
      pk.w = static_cast<uint32_t>(bf16_bits_from_float(v1[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v1[3])) << 16);
      *reinterpret_cast<uint4*>(static_cast<bf16_t*>(out) + gm * n + gn) = pk;
    }
  } else {
    const bool vec = n % 4 == 0;
    for (int c = tid; c < ROWS * (COLS / 4); c += THREADS) {
      const int row = c / (COLS / 4), col = (c % (COLS / 4)) * 4;
      const long gm = m0 + row, gn = n0 + col;
      if (gm >= m || gn >= n) continue;
      const floatx4 v = *reinterpret_cast<const floatx4*>(patch + row * kStride + col);
      const long o = gm * n + gn;
      if (vec) {
        if constexpr (EPI == kStoreBf16) {
          uint2 pk;
          pk.x = static_cast<uint32_t>(bf16_bits_from_float(v[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
          pk.y = static_cast<uint32_t>(bf16_bits_from_float(v[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
          *reinterpret_cast<uint2*>(static_cast<bf16_t*>(out) + o) = pk;
        } else if constexpr (EPI == kStoreF32) {
          *reinterpret_cast<floatx4*>(static_cast<float*>(out) + o) = v;
        } else {
          floatx4* dst = reinterpret_cast<floatx4*>(static_cast<float*>(out) + o);
          const floatx4 old = *dst;
          *dst = floatx4{old[0] + v[0], old[1] + v[1], old[2] + v[2], old[3] + v[3]};
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (gn + e >= n) break;
          if constexpr (EPI == kStoreBf16) static_cast<bf16_t*>(out)[o + e] = from_float<bf16_t>(v[e]);
          else if constexpr (EPI == kStoreF32) static_cast<float*>(out)[o + e] = v[e];
          else static_cast<float*>(out)[o + e] += v[e];
        }
      }
    }
  }
}

// The q|k|v epilogue: THREADS threads take ROWS x COLS floats (stride COLS + 4) from LDS, eight neighbouring columns a
// thread -- a block's eight dimensions, or their eight partners -- rotate them with what lies eight columns away in
// the patch, and store queries to out [m, n_heads * head_dim], keys and values into their pages.
template <int THREADS, int ROWS, int COLS>
__device__ inline void store_patch_rope(const float* patch, bf16_t* __restrict__ out, int m, int n, long m0, long n0, int tid,
                                        const RopeKvArgs& ra) {
  constexpr int kStride = COLS + 4;
  const int d = ra.head_dim;
  if (ra.fragment_order && n0 >= static_cast<long>(ra.n_heads + ra.n_kv_heads) * d) {
    // A patch of value columns only, for a cache in fragment order, where four consecutive tokens of one dimension
    // lie side by side: a thread takes one column of four rows, and where those four tokens' places are four in a
    // row from a multiple of four on (a prompt portion's usually are) it stores them at once.
    static_assert(ROWS % 4 == 0, "rows in fours");
    for (int c = tid; c < (ROWS / 4) * COLS; c += THREADS) {
      const int col = c % COLS, row = (c / COLS) * 4;
      const long gm = m0 + row, gn = n0 + col;
      if (gm >= m || gn >= n) continue;
      const int head = static_cast<int>(gn / d) - ra.n_heads - ra.n_kv_heads, dim = static_cast<int>(gn % d);
      const int rows = static_cast<int>(min(4L, m - gm));
      int slot[4];
      uint16_t bits[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        slot[e] = e < rows ? ra.slot_map[gm + e] : -1;
        bits[e] = bf16_bits_from_float(patch[(row + e) * kStride + col]);
      }
      if (rows == 4 && slot[0] % 4 == 0 && slot[1] == slot[0] + 1 && slot[2] == slot[0] + 2 && slot[3] == slot[0] + 3) {
        const long page = slot[0] / ra.page_tokens;
        const int off = slot[0] % ra.page_tokens;
        bf16_t* region = ra.v_cache + (page * ra.n_kv_heads + head) * static_cast<long>(d) * ra.page_tokens;
        uint2 pk;
        pk.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
        pk.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
        *reinterpret_cast<uint2*>(region + frag_v_offset(off, dim, d)) = pk;
      } else {
        for (int e = 0; e < rows; ++e) {
          const long page = slot[e] / ra.page_tokens;
          const int off = slot[e] % ra.page_tokens;
          bf16_t* region = ra.v_cache + (page * ra.n_kv_heads + head) * static_cast<long>(d) * ra.page_tokens;
          region[frag_v_offset(off, dim, d)].bits = bits[e];
        }
      }
    }
    return;
  }
  for (int c = tid; c < ROWS * (COLS / 8); c += THREADS) {
    const int row = c / (COLS / 8), col = (c % (COLS / 8)) * 8;
    const long gm = m0 + row, gn = n0 + col;
    if (gm >= m || gn >= n) continue;
    const int head = static_cast<int>(gn / d), dim = static_cast<int>(gn % d);
    const bool is_q = head < ra.n_heads, is_v = head >= ra.n_heads + ra.n_kv_heads;
    if (!is_q && !ra.write_kv) continue;
    float v[8];
    {
      const floatx4 v0 = *reinterpret_cast<const floatx4*>(patch + row * kStride + col);
      const floatx4 v1 = *reinterpret_cast<const floatx4*>(patch + row * kStride + col + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = v0[e], v[4 + e] = v1[e];
    }
    if (ra.table != nullptr && !is_v) {
      const bool first = dim % 16 < 8;                       // a block's eight first halves of pairs; their partners lie 8 further
      const float* partner = patch + row * kStride + (first ? col + 8 : col - 8);
      const floatx4 o0 = *reinterpret_cast<const floatx4*>(partner), o1 = *reinterpret_cast<const floatx4*>(partner + 4);
      const floatx4* cs = reinterpret_cast<const floatx4*>(ra.table + gm * (d / 2) + (dim / 16) * 8);   // (cos, sin) of two pairs each
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const floatx4 a = cs[e];
        const float p0 = e < 2 ? o0[2 * e] : o1[2 * e - 4], p1 = e < 2 ? o0[2 * e + 1] : o1[2 * e - 3];
        v[2 * e] = first ? v[2 * e] * a[0] - p0 * a[1] : v[2 * e] * a[0] + p0 * a[1];
        v[2 * e + 1] = first ? v[2 * e + 1] * a[2] - p1 * a[3] : v[2 * e + 1] * a[2] + p1 * a[3];
      }
    }
    uint4 pk;
    pk.x = static_cast<uint32_t>(bf16_bits_from_float(v[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
    pk.y = static_cast<uint32_t>(bf16_bits_from_float(v[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
    pk.z = static_cast<uint32_t>(bf16_bits_from_float(v[4])) | (static_cast<uint32_t>(bf16_bits_from_float(v[5])) << 16);
    pk.w = static_cast<uint32_t>(bf16_bits_from_float(v[6])) | (static_cast<uint32_t>(bf16_bits_from_float(v[7])) << 16);
    if (is_q) {
      *reinterpret_cast<uint4*>(out + gm * (static_cast<long>(ra.n_heads) * d) + gn) = pk;
      continue;
    }
    const int slot = ra.slot_map[gm];
    const long page = slot / ra.page_tokens;
    const int off = slot % ra.page_tokens;
    if (!is_v) {      // keys: [page][kv head][token][dim], or in fragment order: eight dimensions of 16 tokens together
      bf16_t* region = ra.k_cache + (page * ra.n_kv_heads + (head - ra.n_heads)) * ra.page_tokens * d;
      bf16_t* dst = ra.fragment_order ? region + frag_k_offset(off, dim, d) : region + static_cast<long>(off) * d + dim;
      *reinterpret_cast<uint4*>(dst) = pk;
    } else {          // values are kept transposed: [page][kv head][dim][token], or in fragment order
      bf16_t* region = ra.v_cache + (page * ra.n_kv_heads + (head - ra.n_heads - ra.n_kv_heads)) * static_cast<long>(d) * ra.page_tokens;
      bf16_t* dst = ra.fragment_order ? region + frag_v_offset(off, dim, d) : region + static_cast<long>(dim) * ra.page_tokens + off;
      const long step = ra.fragment_order ? 4 : ra.page_tokens;
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e * step] = from_float<bf16_t>(v[e]);
    }
  }
}

// ---- operands through registers ---------------------------------------------------------------
// A workgroup of 4 waves computes a 128 x 128 tile.  A tile of each operand is staged in LDS as
// [128 rows][64 k] with rows padded to 144 bytes (which makes the 16-byte fragment reads of
// consecutive lanes cover all banks), in two buffers: while the waves feed MFMAs from one, the next
// k-step is written to the other and the one after it is in flight from memory, in registers.
// Each wave owns a 64 x 64 quarter (2 x 2 MFMA blocks).  Rows, columns and k beyond the matrix are
// read as zero.
struct StagedTile {
  bf16_t a[kBM][kLdsStride];
  bf16_t w[kBN][kLdsStride];
};

template <int EPI>
__global__ __launch_bounds__(256, 2) void gemm_mfma_staged_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, void* __restrict__ out, int m, int n, int k,
    int m_blocks, int n_blocks) {
  constexpr int SETS = 2, kRows = kBM, kThreads = 256;   // SETS register sets: SETS - 1 k-steps in flight while one is written
  constexpr int kChunkRows = kThreads / 8;           // rows one chunk of a thread's loads covers
  constexpr int kChunksA = kRows / kChunkRows, kChunksW = kBN / kChunkRows;
  typedef StagedTile Tile;
  __shared__ __align__(16) unsigned char lds_raw[sizeof(Tile) * 2];
  Tile* tiles = reinterpret_cast<Tile*>(lds_raw);
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave / 2, wn = wave % 2;   // this wave's 64 x 64 part

  int bm, bn;
  tile_of(blockIdx.x, m_blocks, n_blocks, bm, bn);
  const long m0 = static_cast<long>(bm) * kRows, n0 = static_cast<long>(bn) * kBN;

  // global -> LDS: a tile's rows are 8 segments of 16 bytes; thread t moves segment t%8 of rows
  // t/8 + kChunkRows * i (chunk i of each operand; chunks 0..3 carry both where both have as many).
  const int seg = tid % 8, lrow = tid / 8;
  struct Staged {
    uint4 a[kChunksA], w[kChunksW];
  };
  const bf16_t* arow[kChunksA];
  const bf16_t* wrow[kChunksW];
  bool a_ok[kChunksA], w_ok[kChunksW];
#pragma unroll
  for (int i = 0; i < kChunksA; ++i) {
    const long gm = m0 + lrow + kChunkRows * i;
    a_ok[i] = gm < m;
    arow[i] = a + (a_ok[i] ? gm : 0) * k + seg * 8;
  }
#pragma unroll
  for (int i = 0; i < kChunksW; ++i) {
    const long gn = n0 + lrow + kChunkRows * i;
    w_ok[i] = gn < n;
    wrow[i] = w + (w_ok[i] ? gn : 0) * k + seg * 8;
  }
  static_assert(kChunksA == 4, "the loop below moves four chunks a k-step");
  auto load_chunk = [&](Staged& r, int kt, int i) {
    const int kk = kt * kBK;
    const bool k_ok = kk + seg * 8 < k;
    r.a[i] = (k_ok && a_ok[i]) ? load16(arow[i] + kk) : zero16();
    if (i < kChunksW) r.w[i] = (k_ok && w_ok[i]) ? load16(wrow[i] + kk) : zero16();
  };
  auto store_chunk = [&](const Staged& r, int buf, int i) {
    *reinterpret_cast<uint4*>(&tiles[buf].a[lrow + kChunkRows * i][seg * 8]) = r.a[i];
    if (i < kChunksW) *reinterpret_cast<uint4*>(&tiles[buf].w[lrow + kChunkRows * i][seg * 8]) = r.w[i];
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frow = lane % 32, fk = (lane / 32) * 8;

  // Step s of k lives in register set s % SETS on its way from memory.  Iteration t multiplies
  // step t from LDS buffer t % 2; before its MFMAs the wave asks memory for step t + SETS (into the
  // set that step t left in the iteration before), and between its MFMAs it writes step t + 1 to
  // the other buffer, chunk by chunk -- so the memory pipeline, LDS and the matrix cores work at the
  // same time inside one wave, and no register is loaded in the iteration that stores it.
  // (The loop is unrolled over SETS sets x 2 buffers.)
  const int nk = (k + kBK - 1) / kBK;
  Staged r[SETS];
#pragma unroll
  for (int s = 0; s < SETS; ++s)
    if (s < nk) {
#pragma unroll
      for (int i = 0; i < 4; ++i) load_chunk(r[s], s, i);
    }
#pragma unroll
  for (int i = 0; i < 4; ++i) store_chunk(r[0], 0, i);
  if (nk > SETS) {
#pragma unroll
    for (int i = 0; i < 4; ++i) load_chunk(r[0], SETS, i);
  }
  lds_barrier();
  constexpr int kUnroll = SETS % 2 ? 2 * SETS : SETS;
  for (int kt = 0; kt < nk; kt += kUnroll) {
#pragma unroll
    for (int j = 0; j < kUnroll; ++j) {
      const int t = kt + j;
      if (t >= nk) break;
      const int cur = j % 2;
      const bool st = t + 1 < nk;
      // all the k-step's fragments are asked for at once: LDS answers in order, so the MFMAs of the
      // first slice start when its four reads are back while the other twelve are on their way
      uint4 fa[kBK / 16][2], fw[kBK / 16][2];
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          fa[ks][i] = *reinterpret_cast<const uint4*>(&tiles[cur].a[wm * 64 + i * 32 + frow][ks * 16 + fk]);
          fw[ks][i] = *reinterpret_cast<const uint4*>(&tiles[cur].w[wn * 64 + i * 32 + frow][ks * 16 + fk]);
        }
      __builtin_amdgcn_sched_group_barrier(0x100, 16, 0);   // the 16 LDS reads first
#pragma unroll
      for (int ks = 0; ks < kBK / 16; ++ks)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) acc[i][jj] = mfma_32x32x16(fa[ks][i], fw[ks][jj], acc[i][jj]);
      __builtin_amdgcn_sched_group_barrier(0x008, 16, 0);   // then the 16 MFMAs
      if (st) {
#pragma unroll
        for (int i = 0; i < 4; ++i) store_chunk(r[(j + 1) % SETS], 1 - cur, i);
      }
      if (t + 1 + SETS < nk) {
#pragma unroll
        for (int i = 0; i < 4; ++i) load_chunk(r[(j + 1) % SETS], t + 1 + SETS, i);
      }
      lds_barrier();
    }
  }

  // The tile goes out through LDS (as float [128][128 + 4]), so that a thread stores four
  // neighbouring columns of a row at once.  acc[i][j][r] is row wm*64 + i*32 + 8*(r/4) + 4*(lane/32)
  // + r%4 and column wn*64 + j*32 + lane%32 of the tile.
  constexpr int kOutStride = kBN + 4;
  static_assert(sizeof(float) * kBM * kOutStride <= sizeof(Tile) * 2, "the output tile must fit the operand buffers");
  float* tile_out = reinterpret_cast<float*>(lds_raw);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        tile_out[(wm * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4) * kOutStride + wn * 64 + j * 32 + lane % 32] =
            acc[i][j][r];
  lds_barrier();
  store_patch<EPI, kThreads, kBM, kBN>(tile_out, out, m, n, m0, n0, tid);
}

// ---- operands straight into LDS ---------------------------------------------------------------
// The same product with the operand tiles going from memory into LDS without passing registers
// (global_load_lds_dwordx4: a wave's 64 lanes bring 16 bytes each to 1 KB of consecutive LDS), in a
// ring of STAGES buffers: step t + STAGES - 1 is asked for when step t's multiplication starts, one
// barrier a step.  No registers are spent on staging and no instruction on writing LDS, so twice
// the waves fit a CU, and the forms below are 15-30 % faster than those above on every shape measured
// (2048 x 11264 x 2048: 104 against 131 us; 2048 x 2048 x 5632: 52 against 74; 4096^3: 1,139 against
// 1,015 TFLOP/s).  What did not help: a deeper ring where the tiles fill the chip (three stages are
// slower than two; with fewer tiles than CUs a step is as long as a load takes, and four stages of a
// 64 x 64 tile halve that: 512 x 2048 x 5632 48 -> 28 us), raising the waves' priority around the MFMAs, 128 x 64 parts for a wave with half the waves.
//
// The weight comes packed (the weight-streaming kernel's order) and its blocks are copied as they are: see the
// kernel.  The rows of x lie in LDS without padding, BK * 2 bytes each; the 16-byte segment s of row r lies in
// slot s ^ key(r) of its row, key(r) = (r / 2) % 8 for rows of 128 bytes and r % 16 for rows of 256.  A
// fragment read is served sixteen lanes (rows r .. r + 15, one segment) at a time from 64 banks of
// four bytes: two rows of 128 bytes share the banks' span, so the eight rows of one parity must lie
// in eight different slots (with r % 8 as the key rows r and r + 8 met in one bank: counted, half of
// all LDS cycles were conflicts).  A wave-wide load covers 1024 / (BK * 2) rows; which segment a lane
// brings follows from where its 16 bytes land.
//
// WM x WN waves take TM x TN MFMA blocks of 32 x 32 each.  An output element is added up over k in
// ascending order, as in the form above: the same bits whichever form the shape selects.
// k must be a multiple of BK; rows beyond m are read from the last row, blocks beyond n from the last block, and
// not stored.
template <int PER, int MAX>
__device__ inline void wait_for_stage(int later) {
  if constexpr (MAX == 0) {
    wait_loads<0>();
  } else {
    if (later >= MAX) wait_loads<PER * MAX>();
    else wait_for_stage<PER, MAX - 1>(later);
  }
}

template <int ROW_BYTES>
__device__ inline int slot_key(int row) {
  return ROW_BYTES == 128 ? (row >> 1) & 7 : row & 15;
}

template <int WM, int WN, int TM, int TN, int BK, int STAGES>
struct DirectShape {
  static constexpr int kRowsA = 32 * TM * WM, kRowsW = 32 * TN * WN, kRowBytes = BK * 2;
  static constexpr int kWaves = WM * WN, kThreads = 64 * kWaves;
  static constexpr int kStageBytes = (kRowsA + kRowsW) * kRowBytes;
  static constexpr int kPatchBytes = 32 * (32 * TN + 4) * 4;                   // a wave's 32 rows of output, as floats
  static constexpr int kLdsBytes = STAGES * kStageBytes > kWaves * kPatchBytes ? STAGES * kStageBytes : kWaves * kPatchBytes;
  static_assert(kLdsBytes <= 160 * 1024, "a workgroup's LDS");
  static_assert(kRowBytes == 128 || kRowBytes == 256, "rows of 128 or 256 bytes (the slot rule)");
};

template <int EPI, int WM, int WN, int TM, int TN, int BK, int STAGES, int MINWG>
__global__ __launch_bounds__(64 * WM * WN, MINWG) void gemm_mfma_direct_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, void* __restrict__ out, int m, int n, int k, int m_blocks,
    int n_blocks, const RopeKvArgs ra, const RowScaleArgs rows) {
  typedef DirectShape<WM, WN, TM, TN, BK, STAGES> S;
  constexpr int RA = S::kRowsA, RW = S::kRowsW, RB = S::kRowBytes, NW = S::kWaves;
  constexpr int kGroupRows = 1024 / RB;                    // rows a wave-wide load covers
  constexpr int GA = RA / kGroupRows, GW = RW / kGroupRows, PER = (GA + GW + NW - 1) / NW;
  extern __shared__ __align__(1024) unsigned char direct_lds[];
  const unsigned lds_base = static_cast<unsigned>(
      reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char*)direct_lds));   // its LDS address
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN, wn = wave % WN;
  int bm, bn;
  tile_of(blockIdx.x, m_blocks, n_blocks, bm, bn);
  const long m0 = static_cast<long>(bm) * RA, n0 = static_cast<long>(bn) * RW;
  // gridDim.y > 1: k is cut into that many equal parts (each whole steps), and part y's sums go to an output of
  // its own, out + y * m * n (the plain store epilogues only: whoever reads them adds the parts up in order)
  const int nk = k / BK / static_cast<int>(gridDim.y);
  const size_t k_first = static_cast<size_t>(blockIdx.y) * nk * RB;       // in bytes of a row
  if constexpr (EPI == kStoreF32) out = static_cast<float*>(out) + static_cast<size_t>(blockIdx.y) * m * n;
  // The weight comes in the order the weight-streaming kernel reads, so that a model keeps every weight once:
  // [n / 16][k / 32][64 lanes][8] -- blocks of 16 rows x 32 k, 1 KB each, the 16 bytes of row r and k 8 c .. 8 c + 7 at
  // ((r / 16) * (k / 32) + c / 4) * 1024 + ((c % 4) * 16 + r % 16) * 16 (rows beyond n are zeros).  A wave-wide load
  // brings one such block, 1 KB of consecutive memory to 1 KB of consecutive LDS, and the weight's part of a stage is
  // the tile's blocks as they lie in memory, [rows / 16][BK / 32][1 KB]: a fragment read (lane l: row l % 32, k-slot
  // l / 32) takes 16 consecutive rows' 16 bytes side by side, 256 bytes without a bank conflict, and its address is the
  // lane's own offset plus a constant for the slice (no key to fold in, as the rows of x need).
  static_assert(BK % 32 == 0 && RW % 16 == 0, "whole blocks of the packed weight");
  constexpr int kBlocksK = BK / 32;                              // blocks a row block brings every step
  constexpr size_t kPackedStep = static_cast<size_t>(kBlocksK) * 1024;
  static_assert(GW == RW / 16 * kBlocksK, "a wave-wide load of the weight is one block");
  const long w_row_blocks = (static_cast<long>(n) + 15) / 16;

  // the groups of rows (of x) and the blocks (of w) this wave brings every step (a spare turn repeats the last: the
  // same bytes to the same place), and which of a row's segments this lane's 16 bytes of x are
  const int lr = (lane * 16) / RB, ls = (lane * 16 % RB) / 16;
  const unsigned char* src[PER];
  unsigned dst[PER];
  bool piece_of_w[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    int g = wave + NW * i;
    if (g >= GA + GW) g = GA + GW - 1;
    const bool of_a = g < GA;
    if (of_a) {
      const int trow = g * kGroupRows + lr;
      const int seg = ls ^ slot_key<RB>(trow);
      long row = m0 + trow;
      if (row > m - 1) row = m - 1;
      src[i] = reinterpret_cast<const unsigned char*>(a + row * k) + k_first + seg * 16;
      dst[i] = g * 1024;
    } else {
      const int gw = g - GA;
      long block = n0 / 16 + gw / kBlocksK;
      if (block > w_row_blocks - 1) block = w_row_blocks - 1;
      src[i] = reinterpret_cast<const unsigned char*>(w) +
               (block * (k / 32) + static_cast<long>(blockIdx.y) * nk * kBlocksK + gw % kBlocksK) * 1024 + lane * 16;
      dst[i] = RA * RB + gw * 1024;
    }
    piece_of_w[i] = !of_a;                  // (the same in all lanes of the wave)
  }
  auto ask = [&](int step) {
    const unsigned base = lds_base + (step % STAGES) * S::kStageBytes;
    const size_t at_a = static_cast<size_t>(step) * RB, at_w = static_cast<size_t>(step) * kPackedStep;   // once a step
#pragma unroll
    for (int i = 0; i < PER; ++i)
      load_to_lds_16(src[i] + (piece_of_w[i] ? at_w : at_a), __builtin_amdgcn_readfirstlane(base + dst[i]));
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < nk) ask(s);

  // kSwigluScaledBf16: the tile's rows' sums of squares from their parts, a chain a thread (its loads all in flight
  // together), beside the first operands' way into LDS.  (The compiler's wait for these loads knows nothing of the
  // operands asked for before them and so waits for those too: loads return in the order asked.  By the loop's own
  // waits, which count the operands' loads alone, these are done.)
  __shared__ __align__(16) float part_sum[EPI == kSwigluScaledBf16 ? kPartSums * RA : 4];
  if constexpr (EPI == kSwigluScaledBf16) {
    static_assert(kPartSums * RA % S::kThreads == 0 && kPartSums * RA / 4 <= S::kThreads, "whole chains a thread");
    constexpr int kAhead = 16;              // parts of a chain asked for together: one way to memory and back for 128 parts
    // Four rows a thread where the parts' rows allow loads of 16 bytes (a tile begins at a multiple of 64 rows): a CU
    // takes a wave's load every 19 clocks or so, whatever its width, and a row a thread was 128 of them a tile of 64
    // rows and 128 parts -- a microsecond, with the operands' loads waiting among them.
    if (rows.stride % 4 == 0 && reinterpret_cast<uintptr_t>(rows.parts) % 16 == 0) {
      if (tid < kPartSums * RA / 4) {
        const int row = (tid % (RA / 4)) * 4, chain = tid / (RA / 4);
        const bool live = m0 + row < m;     // (then all four are within the stride, which is no less than m)
        const float* p = rows.parts + (live ? m0 + row : 0);
        floatx4 ss = {0.f, 0.f, 0.f, 0.f};
        for (int b0 = chain; b0 < rows.blocks; b0 += kAhead * kPartSums) {
          floatx4 part[kAhead];
#pragma unroll
          for (int i = 0; i < kAhead; ++i) {
            const int b = b0 + i * kPartSums;
            part[i] = live && b < rows.blocks ? *reinterpret_cast<const floatx4*>(p + static_cast<long>(b) * rows.stride)
                                              : floatx4{0.f, 0.f, 0.f, 0.f};
          }
#pragma unroll
          for (int i = 0; i < kAhead; ++i) ss += part[i];        // (in ascending order; a part that is not there adds 0)
        }
        *reinterpret_cast<floatx4*>(part_sum + chain * RA + row) = ss;
      }
    } else
#pragma unroll
    for (int turn = 0; turn < kPartSums * RA / S::kThreads; ++turn) {
      const int slot = turn * S::kThreads + tid, row = slot % RA, chain = slot / RA;
      const bool live = m0 + row < m;
      const float* p = rows.parts + (live ? m0 + row : 0);
      float ss = 0.f;
      for (int b0 = chain; b0 < rows.blocks; b0 += kAhead * kPartSums) {
        float part[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
          const int b = b0 + i * kPartSums;
          part[i] = live && b < rows.blocks ? p[static_cast<long>(b) * rows.stride] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < kAhead; ++i) ss += part[i];          // (in ascending order; a part that is not there adds 0)
      }
      part_sum[slot] = ss;
    }
  }

  const int frow = lane % 32, fhalf = lane / 32;
  int aoff[TM], woff[TN], aswz[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int r = (wm * TM + i) * 32 + frow;
    aoff[i] = r * RB;
    aswz[i] = slot_key<RB>(r);
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    // row r's place in its block of 16, in the block row's first block of the stage; k-slot fhalf of a slice's two
    const int r = (wn * TN + j) * 32 + frow;
    woff[j] = RA * RB + (r / 16) * (kBlocksK * 1024) + (r % 16) * 16 + fhalf * 256;
  }
  constexpr int kSlices = BK / 16;
  uint4 fa[2][TM], fw[2][TN];
  auto read_fragments = [&](int set, const unsigned char* stage, int slice) {
    const int s = slice * 2 + fhalf;
    // the weight's k-slots 2 slice and 2 slice + 1: block (2 slice) / 4 of the row block, 256 bytes a slot in it
    const int w_slice = (slice / 2) * 1024 + (slice % 2) * 512;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[set][i] = *reinterpret_cast<const uint4*>(stage + aoff[i] + ((s ^ aswz[i]) * 16));
#pragma unroll
    for (int j = 0; j < TN; ++j) fw[set][j] = *reinterpret_cast<const uint4*>(stage + woff[j] + w_slice);
  };

  for (int t = 0; t < nk; ++t) {
    // step t has landed once only the steps asked for after it are outstanding
    wait_for_stage<PER, STAGES - 2>(min(nk - 1, t + STAGES - 2) - t);
    lds_barrier();          // everybody's part of step t is there, and nobody reads step t - 1 any more
    if (t + STAGES - 1 < nk) ask(t + STAGES - 1);
    const unsigned char* stage = direct_lds + (t % STAGES) * S::kStageBytes;
    read_fragments(0, stage, 0);
    __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
    for (int ks = 0; ks < kSlices; ++ks) {
      // the next slice's fragments are asked for before this slice's MFMAs, which hide the wait (the
      // order is pinned: left alone, the compiler moves the reads down to where their registers come free)
      if (ks + 1 < kSlices) {
        read_fragments((ks + 1) % 2, stage, ks + 1);
        __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = mfma_32x32x16(fa[ks % 2][i], fw[ks % 2][j], acc[i][j]);
      __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
    }
  }
  lds_barrier();            // the last step has been read: LDS is free for the output

  // The tile goes out through LDS so that a thread stores four neighbouring columns of a row at once:
  // every wave for itself, 32 rows of its part at a time through a patch of its own (no barrier).
  // acc[i][j][r] is row i 32 + 8 (r / 4) + 4 (lane / 32) + r % 4 and column j 32 + lane % 32 of the part.
  constexpr int kStride = 32 * TN + 4;
  float* patch = reinterpret_cast<float*>(direct_lds) + wave * (S::kPatchBytes / 4);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) patch[(8 * (r / 4) + 4 * (lane / 32) + r % 4) * kStride + j * 32 + lane % 32] = acc[i][j][r];
    if constexpr (EPI == kRopeKvBf16)
      store_patch_rope<kWave, 32, 32 * TN>(patch, static_cast<bf16_t*>(out), m, n, m0 + (wm * TM + i) * 32, n0 + wn * TN * 32, lane, ra);
    else if constexpr (EPI == kSwigluScaledBf16)
      store_patch<EPI, kWave, 32, 32 * TN>(patch, out, m, n, m0 + (wm * TM + i) * 32, n0 + wn * TN * 32, lane,
                                           RowScale{part_sum + (wm * TM + i) * 32, RA, 1.0f / static_cast<float>(k), rows.eps});
    else
      store_patch<EPI, kWave, 32, 32 * TN>(patch, out, m, n, m0 + (wm * TM + i) * 32, n0 + wn * TN * 32, lane);
  }
}

template <int EPI, int WM, int WN, int TM, int TN, int BK, int STAGES, int MINWG>
int launch_direct(const bf16_t* ap, const bf16_t* wp, void* out, int m, int n, int k, hipStream_t s, const RopeKvArgs& ra,
                  int k_parts = 1, const RowScaleArgs& rows = RowScaleArgs{}) {
  typedef DirectShape<WM, WN, TM, TN, BK, STAGES> S;
  auto kernel = gemm_mfma_direct_kernel<EPI, WM, WN, TM, TN, BK, STAGES, MINWG>;
  static bool raised = false;   // per instantiation: allow more than the default dynamic LDS
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            S::kLdsBytes) != hipSuccess)
      return fail("gemm_mfma: cannot raise the dynamic LDS limit");
    raised = true;
  }
  const long m_blocks = (m + S::kRowsA - 1) / S::kRowsA, n_blocks = (n + S::kRowsW - 1) / S::kRowsW;
  kernel<<<dim3(static_cast<unsigned>(m_blocks * n_blocks), static_cast<unsigned>(k_parts)), dim3(S::kThreads), S::kLdsBytes, s>>>(
      ap, wp, out, m, n, k, static_cast<int>(m_blocks), static_cast<int>(n_blocks), ra, rows);
  return 0;
}

// Which tile: the one with which the busiest CU finishes first.  A CU's tiles take their FLOPs over what
// a CU sustains with that tile (TFLOP/s per CU, measured on shapes that fill the chip), and no tile is
// faster than its k-steps follow each other when nothing else hides their latency (microseconds a step,
// measured on shapes with fewer tiles than CUs: the small tile with four stages is for those).  A
// function of (m, n, k) alone; every tile adds over k in the same order.
// The rates are measured with the weights coming from memory, as they do inside a model (the caches filled
// with other data before each run, then the activations and the output touched): a loop over one product
// finds its weights in the 256 MB cache before memory and flatters the small tiles and the short rings --
// 128 x 64 with two stages sustains 3.2 TFLOP/s a CU in such a loop and 2.2-2.4 behind a layer's other
// kernels.  So the tiles that leave room in LDS keep more steps in flight: 128 x 128 (eight waves of 64 x 32,
// four stages) took the place of 128 x 64 with two stages and four workgroups a CU, which no shape selects any
// more but the q|k|v product (a product takes 20-29 % less time where it was selected: 2,048 x 2,048 x 5,632 85 -> 65 us), and 256 x 128
// has three stages (5-18 % less than with two).  Five stages for 128 x 128, three for 128 x 64 (then two
// workgroups a CU) and 128 x 128 with four waves of 64 x 64 were no better or worse.
struct DirectForm {
  int rows, cols;
  double tflops_a_cu, us_a_step;
};
// The last, 128 x 64 with two stages and four workgroups a CU, is for the q|k|v epilogue alone: what comes after the
// loop is long there (rotation, three destinations), and several workgroups a CU run it beside each other's loops
// (a 2,048-token TinyLlama prompt 1 % faster with it than with 160 tiles of 256 x 128, both libraries in one process).
constexpr int kDirectForms = 6;
constexpr DirectForm kDirectForm[kDirectForms] = {
    {256, 256, 4.45, 0.5}, {256, 192, 3.9, 0.5}, {256, 128, 3.8, 0.5}, {128, 128, 3.1, 0.5}, {64, 64, 2.2, 0.28}, {128, 64, 2.9, 0.5}};

int direct_form(int m, int n, int k, bool long_epilogue) {
  int best = 0;
  double best_time = 0.0;
  for (int f = 0; f < (long_epilogue ? kDirectForms : kDirectForms - 1); ++f) {
    const DirectForm& form = kDirectForm[f];
    const long tiles = static_cast<long>((m + form.rows - 1) / form.rows) * ((n + form.cols - 1) / form.cols);
    const long turns = (tiles + compute_units() - 1) / compute_units();
    const double work = turns * (2.0e-6 * form.rows * form.cols * k) / form.tflops_a_cu;
    const double chain = 3.0 + (k / 64) * form.us_a_step;
    const double time = work > chain ? work : chain;
    if (f == 0 || time < best_time) best = f, best_time = time;
  }
  return best;
}

template <int EPI>
int launch_direct_form(const bf16_t* ap, const bf16_t* wp, void* out, int m, int n, int k, hipStream_t s,
                       const RopeKvArgs& ra = RopeKvArgs{}, const RowScaleArgs& rows = RowScaleArgs{}) {
  switch (direct_form(m, n, k, EPI == kRopeKvBf16)) {
    case 0: return launch_direct<EPI, 4, 4, 2, 2, 64, 2, 1>(ap, wp, out, m, n, k, s, ra, 1, rows);
    case 1: return launch_direct<EPI, 4, 2, 2, 3, 64, 2, 1>(ap, wp, out, m, n, k, s, ra, 1, rows);
    case 2: return launch_direct<EPI, 4, 2, 2, 2, 64, 3, 1>(ap, wp, out, m, n, k, s, ra, 1, rows);
    case 3: return launch_direct<EPI, 2, 4, 2, 1, 64, 4, 1>(ap, wp, out, m, n, k, s, ra, 1, rows);
    case 5: return launch_direct<EPI, 2, 2, 2, 1, 64, 2, 4>(ap, wp, out, m, n, k, s, ra, 1, rows);
    default: return launch_direct<EPI, 2, 2, 1, 1, 64, 4, 2>(ap, wp, out, m, n, k, s, ra, 1, rows);
  }
}

bool direct_operands(const void* ap, const void* wp, int k) {
  // operands straight into LDS wherever k is whole steps of it and rows start on 16-byte boundaries
  return k % 64 == 0 && reinterpret_cast<uintptr_t>(ap) % 16 == 0 && reinterpret_cast<uintptr_t>(wp) % 16 == 0;
}

// w_packed: the weight in the weight-streaming kernel's order, for the kernel with operands straight into LDS (k in
// whole steps of 64, operands on 16-byte boundaries); else the weight by rows, for the kernel that stages its tiles
// through registers (any k that is a multiple of 8).
template <int EPI>
int launch_tiled(const bf16_t* ap, const bf16_t* wp, void* out, int m, int n, int k, hipStream_t s, int w_packed) {
  if (w_packed) {
    if (!direct_operands(ap, wp, k))
      return fail("gemm_mfma: a packed weight needs k in whole steps of 64 and operands on 16-byte boundaries (K=%d)", k);
    return launch_direct_form<EPI>(ap, wp, out, m, n, k, s);
  }
  const long m_blocks = (m + kBM - 1) / kBM, n_blocks = (n + kBN - 1) / kBN;
  gemm_mfma_staged_kernel<EPI><<<dim3(static_cast<unsigned>(m_blocks * n_blocks)), dim3(256), 0, s>>>(
      ap, wp, out, m, n, k, static_cast<int>(m_blocks), static_cast<int>(n_blocks));
  return 0;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_gemm_mfma(const void* a, const void* w, int w_packed, void* out, int epilogue, int m, int n, int k,
                              void* stream) {
  BC4G_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 8 == 0, "gemm_mfma: K=%d must be a positive multiple of 8 (M=%d N=%d)",
               k, m, n);
  if (m == 0) return 0;
  BC4G_REQUIRE(((m + 63L) / 64) * ((n + 63L) / 64) <= 2147483647L, "gemm_mfma: too many tiles");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bf16_t* ap = static_cast<const bf16_t*>(a);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  int e = 0;
  switch (epilogue) {
    case kStoreBf16: e = launch_tiled<kStoreBf16>(ap, wp, out, m, n, k, s, w_packed); break;
    case kStoreF32: e = launch_tiled<kStoreF32>(ap, wp, out, m, n, k, s, w_packed); break;
    case kAccumF32: e = launch_tiled<kAccumF32>(ap, wp, out, m, n, k, s, w_packed); break;
    case kSwigluBf16:
      BC4G_REQUIRE(n % 16 == 0, "gemm_mfma: SwiGLU needs blocks of eight gate and eight up rows, N=%d is no multiple of 16", n);
      e = launch_tiled<kSwigluBf16>(ap, wp, out, m, n, k, s, w_packed);
      break;
    default: return fail("gemm_mfma: unknown epilogue %d", epilogue);
  }
  if (e) return e;
  return check_launch("gemm_mfma");
}

extern "C" int bc4g_gemm_mfma_swiglu_scaled(const void* a, const float* ssq_parts, int ssq_blocks, int ssq_stride, float eps,
                                            const void* w, int w_packed, void* out, int m, int n, int k, void* stream) {
  BC4G_REQUIRE(m >= 0 && n > 0 && n % 16 == 0 && k > 0 && direct_operands(a, w, k) && w_packed,
               "gemm_mfma_swiglu_scaled: K=%d must be a multiple of 64, N=%d one of 16, the weight packed and the operands on 16-byte boundaries (M=%d)", k, n, m);
  BC4G_REQUIRE(ssq_parts != nullptr && ssq_blocks > 0 && ssq_stride >= m && eps >= 0.f,
               "gemm_mfma_swiglu_scaled: the sums of squares need %d parts of at least %d rows, and eps must not be negative", ssq_blocks, m);
  if (m == 0) return 0;
  BC4G_REQUIRE(((m + 63L) / 64) * ((n + 63L) / 64) <= 2147483647L, "gemm_mfma_swiglu_scaled: too many tiles");
  if (int e = launch_direct_form<kSwigluScaledBf16>(static_cast<const bf16_t*>(a), static_cast<const bf16_t*>(w), out, m, n, k,
                                                     static_cast<hipStream_t>(stream), RopeKvArgs{},
                                                     RowScaleArgs{ssq_parts, ssq_blocks, ssq_stride, eps}))
    return e;
  return check_launch("gemm_mfma_swiglu_scaled");
}

extern "C" int bc4g_gemm_mfma_parts(const void* a, const void* w, int w_packed, float* parts, int m, int n, int k, int k_parts,
                                    void* stream) {
  BC4G_REQUIRE(m > 0 && n > 0 && k > 0 && k_parts >= 1 && k_parts <= 16 && k % (64 * k_parts) == 0 && direct_operands(a, w, k) &&
                   w_packed,
               "gemm_mfma_parts: K=%d must be %d times a multiple of 64, the weight packed and the operands on 16-byte boundaries "
               "(M=%d N=%d)", k, k_parts, m, n);
  BC4G_REQUIRE(((m + 63L) / 64) * ((n + 63L) / 64) <= 2147483647L, "gemm_mfma_parts: too many tiles");
  if (int e = launch_direct<kStoreF32, 2, 2, 1, 1, 64, 4, 2>(static_cast<const bf16_t*>(a), static_cast<const bf16_t*>(w), parts, m, n,
                                                               k, static_cast<hipStream_t>(stream), RopeKvArgs{}, k_parts))
    return e;
  return check_launch("gemm_mfma_parts");
}

extern "C" int bc4g_gemm_mfma_qkv(const void* a, const void* w, int w_packed, void* out, const float* table, const int32_t* slot_map,
                                  void* k_cache, void* v_cache, int m, int n, int k, int n_heads, int n_kv_heads,
                                  int head_dim, int page_tokens, int write_kv, void* stream) {
  BC4G_REQUIRE(m > 0 && n > 0 && k > 0 && direct_operands(a, w, k) && w_packed,
               "gemm_mfma_qkv: K=%d must be a multiple of 64, the weight packed and the operands on 16-byte boundaries (M=%d N=%d)", k, m, n);
  BC4G_REQUIRE(n_heads > 0 && n_kv_heads > 0 && head_dim > 0 && head_dim % 16 == 0 &&
                   static_cast<long>(n_heads + 2 * n_kv_heads) * head_dim == n,
               "gemm_mfma_qkv: %d + 2 x %d heads of %d (a multiple of 16) are not %d columns", n_heads, n_kv_heads, head_dim, n);
  BC4G_REQUIRE(!write_kv || (page_tokens > 0 && k_cache && v_cache && slot_map), "gemm_mfma_qkv: cache write asked for without a cache");
  BC4G_REQUIRE(((m + 63L) / 64) * ((n + 63L) / 64) <= 2147483647L, "gemm_mfma_qkv: too many tiles");
  RopeKvArgs ra{};
  ra.table = reinterpret_cast<const float2*>(table);
  ra.slot_map = slot_map;
  ra.k_cache = static_cast<bf16_t*>(k_cache);
  ra.v_cache = static_cast<bf16_t*>(v_cache);
  ra.n_heads = n_heads;
  ra.n_kv_heads = n_kv_heads;
  ra.head_dim = head_dim;
  ra.page_tokens = page_tokens;
  ra.write_kv = write_kv ? 1 : 0;
  ra.fragment_order = write_kv && cache_fragment_order(true, head_dim, page_tokens) ? 1 : 0;
  if (int e = launch_direct_form<kRopeKvBf16>(static_cast<const bf16_t*>(a), static_cast<const bf16_t*>(w), out, m, n, k,
                                              static_cast<hipStream_t>(stream), ra))
    return e;
  return check_launch("gemm_mfma_qkv");
}

extern "C" int bc4g_gemm_mfma_tile(const void* a, const void* w, int m, int n, int k, int qkv, int* rows, int* cols) {
  BC4G_REQUIRE(rows != nullptr && cols != nullptr && m > 0 && n > 0 && k > 0, "gemm_mfma_tile: sizes and two places for the answer");
  if (direct_operands(a, w, k)) {
    const DirectForm& form = kDirectForm[direct_form(m, n, k, qkv != 0)];
    *rows = form.rows, *cols = form.cols;
  } else {
    *rows = kBM, *cols = kBN;
  }
  return 0;
}
