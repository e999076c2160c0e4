// Causal softmax attention over the paged cache on the matrix cores, bfloat16, for prompt
// portions and decoded tokens alike.
//
// One wave owns a tile of 16 query rows: `tpt` consecutive tokens of one request times `hg`
// query heads that share one key/value head (hg * tpt <= 16).  It walks the keys it may see in
// tiles of 32 and never writes scores to memory:
//   S^T = K Q^T   16x16x32 MFMAs with the keys as rows, so that a lane holds one query row's
//                 scores and the softmax statistics are reductions inside a lane plus two
//                 shuffles;  K comes straight from the cache pages as the A operand (the pages
//                 are stored in the operand's order: a fragment is one contiguous kilobyte)
//   online softmax in float, base 2, masked by absolute position (and the window); the running
//                 maximum is kept over raw scores and the scale enters the exponent's argument
//   O^T += V^T P^T   with P^T taken from the score registers as the B operand and V^T loaded
//                 from the value pages, stored in that operand's order too (8-byte loads of 4
//                 consecutive tokens, the 64 lanes' loads contiguous)
// Prompt portions bring many tiles of one request: there a workgroup is four waves with
// consecutive tiles that walk their keys together (WS == 0) -- a key tile goes from the cache into LDS
// once (a straight copy: the pages are in operand order already; from memory into LDS without passing
// registers) and every wave takes its operands from there, so a key is fetched once for 4 * QT * 16
// query rows; the tiles up to three ahead are in flight during the arithmetic, and there is one
// barrier a tile.  (WS == 1 is
// the same without LDS, four independent waves each fetching its own keys: the simpler form, kept as
// a cross-check -- both give the same bits.)
// Decoded tokens bring few tiles and long key walks: there a workgroup is one tile and its WS
// waves cut the tile's keys between them, then combine their partial results in LDS (in wave
// order).  On top of that, with n_splits > 1 the key range is cut into that many parts over
// workgroups (grid z); each part writes unnormalized float partials, and
// attention_merge_kernel combines them.
//
// A row reads keys max(0, p - window + 1) .. p only.  Keys beyond the tile's last position may
// never have been written: their scores are replaced by -inf and their values by zero, so that
// whatever lies in those places (NaN included) cannot reach the sums.
#include <math.h>

#include <mutex>
#include <type_traits>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kWavesPerBlock = 4;
constexpr float kLog2e = 1.4426950408889634f;

// 2^x by the hardware instruction (arguments here are <= 0 or -inf; results below the smallest
// normal number flush to zero, which is what a softmax weight that small may do).
__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Two floats to two bfloat16 (round to nearest even) in one instruction of gfx950.
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
  uint32_t r;
  asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
  return r;
}

// Maxima in one instruction each.  (fmaxf would first quiet a possible signalling NaN in every operand
// with an instruction of its own; the operands here are MFMA results, -inf or earlier maxima.)
__device__ inline float max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ inline float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// max / sum of a value over the four lanes l, l ^ 16, l ^ 32, l ^ 48, in every lane: the swap
// instructions of gfx950 exchange half-rows between two registers in the vector ALU, with no trip
// through LDS.  swap16(x, x) leaves (x of rows 0,0,2,2 | x of rows 1,1,3,3), swap32 the halves alike.
__device__ inline float max_16_32(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float y = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const uint32_t v = __float_as_uint(y);
  const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ inline float sum_16_32(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float y = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const uint32_t v = __float_as_uint(y);
  const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// What a tile's loads bring for blocks of keys that no row of the walk sees.
__device__ __align__(16) const unsigned char kZeroLine[1024] = {0};     // (a wave's load wide)

struct AttnArgs {
  const bf16_t* qkv;           // queries: row t, head h at qkv + t * q_stride + h * d
  bf16_t* out;                 // [T, n_heads * d]               (n_splits == 1)
  float* part_o;               // [n_splits, T, n_heads, d]      (n_splits > 1), unnormalized
  float* part_ml;              // [n_splits, T, n_heads, 2]      running max (base 2) and sum
  const bf16_t* k_cache;       // [pages, n_kv, P * d], every page and head in fragment order (common.h)
  const bf16_t* v_cache;       // likewise
  const int32_t* block_table;  // [S, table_stride]
  const int32_t* seq_start;    // [S + 1] first row of each request in the batch
  const int32_t* seq_ctx;      // [S] tokens cached before this step
  const int32_t* tile_start;   // [S + 1] first tile of each request
  int table_stride, n_seqs, n_tiles, n_tokens, q_stride;
  int n_heads, n_kv_heads, head_dim, page_tokens, window;
  int hg, tpt, n_sub;          // heads per tile, tokens per tile, head sub-groups per kv head
  int n_splits;
  const int32_t* items;        // prompt form with a work list: workgroup y takes piece items[y] % 2^20, part (items[y] >> 20) % 16 of
                               // items[y] >> 24 parts of that piece's keys (nullptr: the grid's x is the piece, z the part of n_splits)
  const int32_t* row_parts;    // with items: into how many parts each row's keys were cut ([T]; 1: the row is written as it is)
  int single_rows;             // every request brings exactly one row (a decode step): request s is tile s and row s
  float scale_log2;            // softmax scale times log2(e)
};

// DJ: k-steps of 32 over head_dim for the scores; DB: blocks of 16 output dimensions; QT: 16-row
// query tiles per wave (consecutive tokens), which share every key and value fragment the wave
// loads -- prompt portions use 4 (or 2 for large heads), decoded tokens 1.
// WS: 1, or the number of waves that share one tile's keys.
constexpr int kMergePad = 4;   // floats between rows of the partial outputs in LDS

// EXACT: the head size is exactly 16 * DB (the usual sizes 64, 128, 256): no test against it is left.
template <int DJ, int DB, int QT, int WS, bool EXACT>
__global__ __launch_bounds__((WS > 1 ? WS : kWavesPerBlock) * kWave, 2) void attention_mfma_kernel(
    const AttnArgs a) {
  static_assert(WS <= 1 || QT == 1, "waves share a tile's keys for single query tiles only");
  constexpr bool kStaged = WS == 0;
  // WS > 1: [WS][16][d + pad] outputs, [WS][16][2] statistics; WS == 0: a ring of key tiles of 128 * d bytes
  extern __shared__ __align__(16) float merge_raw[];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int col = lane % 16, grp = lane / 16;
  // what tile_start counts: a wave's tiles (WS == 1), or a workgroup's (one tile, or four waves' tiles).
  // Prompt forms without a work list: the last workgroups first -- under the causal mask a request's last
  // rows walk the most keys, and the longest walks should not be the ones that start last -- in every
  // other (head, part of the keys), and the first ones first in those between: workgroups that are a
  // grid's x extent apart tend to share a CU, and so a long walk meets a short one there.
  // With a work list the host has put the longest walks first and says which piece and part this is.
  const bool listed = kStaged && a.items != nullptr;
  const int item = listed ? a.items[blockIdx.y] : 0;
  const int head_block = listed ? blockIdx.x : blockIdx.y;
  const int part = listed ? (item >> 20) & 15 : blockIdx.z;
  const bool last_first = ((blockIdx.y + blockIdx.z) & 1) == 0;
  const int block_x = listed ? (item & 0xfffff) : ((WS > 1 || !last_first) ? blockIdx.x : gridDim.x - 1 - blockIdx.x);
  const int tile = WS == 1 ? block_x * kWavesPerBlock + wave : block_x;
  if (WS == 1 && tile >= a.n_tiles) return;   // (waves are independent there: no barrier below)

  // Which request this tile belongs to, and that request's rows and context.  Up to 63 requests
  // are looked at by one lane each (three loads, all at once, and a vote); more by bisection.
  int s, row0, q_len, ctx, tile0;
  if (a.single_rows) {
    // nothing to look up but the context: the block table, the query and the context are asked for together
    s = tile0 = row0 = tile;
    q_len = 1;
    ctx = a.seq_ctx[tile];
  } else if (a.n_seqs < kWave) {
    const int ts = lane <= a.n_seqs ? a.tile_start[lane] : 0;
    const int ss = lane <= a.n_seqs ? a.seq_start[lane] : 0;
    const int sc = lane < a.n_seqs ? a.seq_ctx[lane] : 0;
    // (read as scalars: everything derived from them -- key ranges, pages, addresses -- stays scalar)
    s = __builtin_amdgcn_readfirstlane(__popcll(__ballot(lane < a.n_seqs && ts <= tile)) - 1);
    tile0 = __builtin_amdgcn_readlane(ts, s);
    row0 = __builtin_amdgcn_readlane(ss, s);
    q_len = __builtin_amdgcn_readlane(ss, s + 1) - row0;
    ctx = __builtin_amdgcn_readlane(sc, s);
  } else {
    int lo_s = 0, hi_s = a.n_seqs - 1;
    while (lo_s < hi_s) {
      const int mid = (lo_s + hi_s + 1) >> 1;
      if (a.tile_start[mid] <= tile) lo_s = mid; else hi_s = mid - 1;
    }
    s = lo_s;
    tile0 = a.tile_start[s];
    row0 = a.seq_start[s];
    q_len = a.seq_start[s + 1] - row0;
    ctx = a.seq_ctx[s];
  }
  // the workgroup's rows (kStaged: four waves' worth) and this wave's among them
  const int tok0_wg = (tile - tile0) * a.tpt * QT * (kStaged ? kWavesPerBlock : 1);
  const int tok0 = tok0_wg + (kStaged ? wave * a.tpt * QT : 0);
  const int ntok = max(0, min(a.tpt * QT, q_len - tok0));     // (0: a wave past the request's rows)
  const int kvh = head_block / a.n_sub, hsub = head_block % a.n_sub;
  const int group = a.n_heads / a.n_kv_heads;
  const int d = EXACT ? 16 * DB : a.head_dim, P = a.page_tokens;
  const int32_t* table = a.block_table + static_cast<long>(s) * a.table_stride;

  // this lane's query row in each tile (as B operand and as owner of one row's statistics)
  const int q_hsub = col % a.hg;
  const int q_head_in_group = hsub * a.hg + q_hsub;
  const int q_head = kvh * group + q_head_in_group;
  const long qkv_stride = a.q_stride;
  int q_tok[QT], q_pos[QT], q_lo[QT];
  bool q_ok[QT];
  uint4 qf[QT][DJ];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    q_tok[t] = t * a.tpt + col / a.hg;
    q_ok[t] = col / a.hg < a.tpt && q_tok[t] < ntok && q_head_in_group < group;
    q_pos[t] = ctx + tok0 + q_tok[t];
    q_lo[t] = (a.window > 0 && q_pos[t] - a.window + 1 > 0) ? q_pos[t] - a.window + 1 : 0;
#pragma unroll
    for (int j = 0; j < DJ; ++j) {
      const int c = 32 * j + 8 * grp;
      qf[t][j] = (q_ok[t] && (EXACT || c < d))
                     ? load16(a.qkv + (row0 + tok0 + q_tok[t]) * qkv_stride + static_cast<long>(q_head) * d + c)
                     : zero16();
    }
  }

  // the wave's own positions (masks), and those of the rows whose keys the walk covers: the
  // wave's, or (kStaged) the four waves' together
  const int pos_min = ctx + tok0, pos_max = ctx + tok0 + ntok - 1;
  const int walk_min = ctx + tok0_wg;
  const int walk_max = kStaged ? ctx + min(q_len, tok0_wg + kWavesPerBlock * a.tpt * QT) - 1 : pos_max;
  const int lo_min = (a.window > 0 && walk_min - a.window + 1 > 0) ? walk_min - a.window + 1 : 0;
  const int kt_first = lo_min / 32, kt_last = walk_max / 32;
  const int n_kt = kt_last - kt_first + 1;
  // Into how many parts this walk is cut: n_splits (times the waves that share a tile's keys), or what
  // the work list says for this piece.
  const int n_parts = listed ? (item >> 24) : a.n_splits * (WS > 1 ? WS : 1);
  const int per_split = (n_kt + n_parts - 1) / n_parts;
  const int kt_begin = kt_first + (part * (WS > 1 ? WS : 1) + (WS > 1 ? wave : 0)) * per_split;
  const int kt_end = min(kt_last + 1, kt_begin + per_split);
  // kStaged: the tiles of the walk that hold keys of this wave's rows
  const int own_lo = (a.window > 0 && pos_min - a.window + 1 > 0) ? pos_min - a.window + 1 : 0;
  const int own_first = own_lo / 32, own_last = ntok > 0 ? pos_max / 32 : -1;

  // per row: the exponents' reference, the sum of the weights, and -- kept beside the reference so that a tile
  // that moves nothing need not work them out -- the shift it makes in the exponent and the score beyond which it moves
  float m_run[QT], l_run[QT], m_shift[QT], m_limit[QT];
  floatx4 o[QT][DB];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    m_run[t] = -INFINITY;
    m_shift[t] = 0.f;
    m_limit[t] = -INFINITY;
    l_run[t] = 0.f;
#pragma unroll
    for (int b = 0; b < DB; ++b) o[t][b] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // Where a tile's pages are.  The forms without LDS staging hold the request's block table across the wave's
  // lanes (entry i in lane i % 64 of register i / 64), so that finding a tile's page is a lane read and not a trip
  // to memory.  The staged form walks many tiles, and every instruction a wave issues for a tile counts there (a
  // wave issues one every four clocks at best: the lane reads, selects and address arithmetic per half tile were a
  // quarter of a tile's time): it copies the walk's part of the table into LDS first (behind the ring of tiles; a
  // walk over more than kLdsEntries pages reads the rest from memory), looks a page up once, when the walk enters it
  // -- the entry asked of LDS one page ahead -- and keeps the page's place in the cache.
  constexpr int kTableRegs = 4;
  int32_t tbl[kTableRegs];
  const int pages_needed = walk_max / P + 1;
  if constexpr (!kStaged) {
#pragma unroll
    for (int r = 0; r < kTableRegs; ++r) {
      const int idx = r * kWave + lane;
      tbl[r] = (idx < pages_needed && idx < a.table_stride) ? table[idx] : 0;
    }
  }
  auto page_of = [&](int page_index) -> long {       // page_index is the same in every lane
    if (page_index >= kTableRegs * kWave) return table[page_index];
    const int at = page_index % kWave, reg = page_index / kWave;
    int32_t v = __builtin_amdgcn_readlane(tbl[0], at);
#pragma unroll
    for (int r = 1; r < kTableRegs; ++r) {
      const int32_t w = __builtin_amdgcn_readlane(tbl[r], at);
      if (reg == r) v = w;
    }
    return v;
  };
  auto place_of = [&](int32_t page) -> long {   // of the page's keys or values of this key/value head, in elements
    return (static_cast<long>(page) * a.n_kv_heads + kvh) * P * static_cast<long>(d);
  };

  // one tile of 32 keys: key fragments (A operand of the scores) and value fragments (A operand
  // of the output), fetched one tile ahead of their use
  struct KeyTile {
    uint4 k[2][kStaged ? 1 : DJ];
    uint2 v[2][kStaged ? 1 : DB];
    bool ok[2];
  };
  // The cache is in fragment order: the 16 keys at next_off of a page are one block of 16 * d
  // elements in which a key fragment is 1 KB and a value fragment 512 bytes, both in lane order --
  // a scalar base (page, key/value head, block) plus the lane's place.  Where the next tile lies in
  // its page is carried along from tile to tile (the wave walks its tiles in order): no division.
  const int k_lane = lane * 8, v_lane = lane * 4;
  int next_page = (kt_begin * 32) / P, next_off = (kt_begin * 32) % P;
  long block_at[2];                              // where the tile's two blocks of 16 keys lie in the cache
  // kStaged: the place of page next_page in the cache, and the table's entry after it (asked for, not yet waited for)
  constexpr int kLdsEntries = 1024;
  int32_t* walk_table = reinterpret_cast<int32_t*>(merge_raw) + (!kStaged ? 0 : (DB <= 8 ? 4 : 2) * 32 * d);     // behind the ring
  long page_at = 0;
  int32_t entry_ahead = 0;
  const int first_page = next_page, last_entry = min(pages_needed, a.table_stride) - 1;
  typedef __attribute__((address_space(3))) int32_t lds_int;
  auto entry = [&](int page_index) -> int32_t {       // page_index is the same in every lane
    const int at = max(0, min(page_index, last_entry) - first_page);     // (an empty part may begin beyond the last page)
    if (__builtin_expect(at >= kLdsEntries, 0)) return __builtin_amdgcn_readfirstlane(table[first_page + at]);
    return __builtin_amdgcn_readfirstlane(((lds_int*)walk_table)[at]);
  };
  if constexpr (kStaged) {
    for (int i = threadIdx.x; i < kLdsEntries && first_page + i <= last_entry; i += kWavesPerBlock * kWave)
      walk_table[i] = table[first_page + i];
    __syncthreads();
    page_at = place_of(entry(next_page));
    entry_ahead = entry(next_page + 1);
  }
  auto locate = [&](bool (&ok)[2], int kt) {    // tiles are located in order, from kt_begin on
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int kb = kt * 32 + 16 * h;
      ok[h] = kb <= walk_max && kb + 15 >= lo_min;
      if constexpr (kStaged) {
        block_at[h] = page_at + next_off * d;   // (a block that no row sees is never read: wherever this points)
      } else {
        const long page = ok[h] ? page_of(next_page) : 0;
        block_at[h] = ((page * a.n_kv_heads + kvh) * P + next_off) * static_cast<long>(d);
      }
      next_off += 16;                           // pages hold a multiple of 16 tokens
      if (next_off >= P) {
        next_off = 0;
        ++next_page;
        if constexpr (kStaged) {
          page_at = place_of(entry_ahead);
          entry_ahead = entry(next_page + 1);
        }
      }
    }
  };
  auto fetch = [&](KeyTile& t, int kt) {
    locate(t.ok, kt);
    if constexpr (!kStaged) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bf16_t* kbase = a.k_cache + block_at[h];
        const bf16_t* vbase = a.v_cache + block_at[h];
#pragma unroll
        for (int j = 0; j < DJ; ++j)
          t.k[h][j] = (t.ok[h] && (EXACT || 32 * j + 8 * grp < d)) ? load16(kbase + 512 * j + k_lane) : zero16();
#pragma unroll
        for (int b = 0; b < DB; ++b)
          t.v[h][b] = (t.ok[h] && (EXACT || 16 * b < d)) ? *reinterpret_cast<const uint2*>(vbase + 256 * b + v_lane)
                                              : make_uint2(0u, 0u);
      }
    }
  };

  // kStaged: a tile in LDS is four segments of 16 * d elements -- keys of its first and second 16
  // tokens, then their values -- each a copy of the block in the cache, brought straight from memory into
  // a ring of kStages tiles (no register and no LDS write is spent on it): the tile kStages - 1 ahead is
  // asked for when a tile's arithmetic starts, which hides the way from memory behind several tiles' work.
  // A thread brings the same 16-byte pieces of every tile: piece c = threadIdx.x + 256 * r lies in segment
  // c / (2 * d) and lands at byte 16 * c of the tile; a wave's 64 pieces are one load.  Pieces beyond the
  // tile (small heads) are whole waves' and are left out; blocks beyond the walk or before the window are
  // brought from a line of zeros.
  constexpr int kStages = !kStaged ? 1 : (DB <= 8 ? 4 : 2);
  constexpr int kPieces = kStaged ? (4 * 2 * 16 * DB + 255) / 256 : 1;    // per thread, for the largest d of this form
  // (With heads of a multiple of 32 -- the sizes built EXACT -- a wave's 64 pieces lie in one segment: their load
  // is one base address for the wave, worked out in scalar registers, plus 16 bytes a lane.)
  constexpr bool kWholeChunks = EXACT && DB % 2 == 0;
  int piece_seg[kPieces], piece_off[kPieces];
  int chunk_seg[kPieces], chunk_off[kPieces];                             // kWholeChunks: the wave's, not the lane's
  int pieces_a_tile = 0;                                                  // this wave's loads per tile
  if constexpr (kStaged) {
#pragma unroll
    for (int r = 0; r < kPieces; ++r) {
      const int c = threadIdx.x + 256 * r, c0 = (wave * kPieces + r) * kWave;   // (whole chunks: a wave's lie side by side)
      piece_seg[r] = c < 8 * d ? c / (2 * d) : -1;
      piece_off[r] = (c % (2 * d)) * 8;
      chunk_seg[r] = c0 / (2 * d);
      chunk_off[r] = (c0 % (2 * d)) * 8;
      if (kWholeChunks || wave * kWave + 256 * r < 8 * d) ++pieces_a_tile;   // (8 * d is a multiple of 128: whole waves)
    }
  }
  bf16_t* tiles = reinterpret_cast<bf16_t*>(merge_raw);
  const unsigned tiles_lds = static_cast<unsigned>(
      reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) float*)merge_raw));   // its LDS address
  auto stage_ask = [&](int kt, int stage) {     // cache -> LDS; tiles are asked for in order, from kt_begin on
    bool ok[2];
    locate(ok, kt);
    if constexpr (kWholeChunks) {
      // the wave's kPieces chunks of 1 KB go side by side: one LDS address for all and one statement for the loads
      // (what is looked up by a run-time index is chosen here, by selects, before that statement)
      const void* from[kPieces];
#pragma unroll
      for (int r = 0; r < kPieces; ++r) {
        const int seg = chunk_seg[r];
        const long block = (seg & 1) ? block_at[1] : block_at[0];
        const bool seen = (seg & 1) ? ok[1] : ok[0];
        const bf16_t* at = (seg >= 2 ? a.v_cache : a.k_cache) + block + chunk_off[r];
        from[r] = seen ? static_cast<const void*>(at) : static_cast<const void*>(kZeroLine);
      }
      load_chunks_to_lds<kPieces>(from, lane * 16u, tiles_lds + stage * (128 * d) + wave * kPieces * 1024);
    } else {
#pragma unroll
      for (int r = 0; r < kPieces; ++r) {
        if (wave * kWave + 256 * r >= 8 * d) continue;
        const unsigned to = __builtin_amdgcn_readfirstlane(tiles_lds + stage * (128 * d) + (wave * kWave + 256 * r) * 16);
        const int seg = piece_seg[r];
        const bf16_t* from = (seg >= 2 ? a.v_cache : a.k_cache) + ((seg & 1) ? block_at[1] : block_at[0]) + piece_off[r];
        const bool seen = (seg & 1) ? ok[1] : ok[0];
        load_to_lds_16(seen ? static_cast<const void*>(from) : static_cast<const void*>(kZeroLine + lane * 16), to);
      }
    }
  };

  // (the fragments of the largest heads leave no room for a second tile)
  constexpr bool kAhead = DB <= 8;
  KeyTile cur, nxt;
  if constexpr (kStaged) {
    // The loads the compiler knows of (the queries) are waited for here, where it sees it: left to itself it waits for
    // them inside the loop, at the first use of a query, with a count of zero -- which would also wait, tile after tile,
    // for the tile that has just been asked for.
    wait_loads<0>();
#pragma unroll
    for (int ahead = 0; ahead < kStages - 1; ++ahead)
      if (kt_begin + ahead < kt_end) stage_ask(kt_begin + ahead, ahead);
  } else {
    if (kAhead && kt_begin < kt_end) fetch(cur, kt_begin);
  }
  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const bf16_t* tile_lds = tiles + ((kt - kt_begin) % kStages) * (64 * d);
    if constexpr (kStaged) {
      // This tile has landed once only the tiles asked for after it are outstanding (loads finish in order).
      // After the barrier everybody's pieces of it are there and nobody reads the tile before it any more,
      // whose place the tile kStages - 1 ahead takes.
      if constexpr (kWholeChunks && kStages == 4) {       // (every wave brings kPieces loads a tile)
        if (kt + 2 < kt_end) wait_loads<2 * kPieces>();
        else if (kt + 1 < kt_end) wait_loads<kPieces>();
        else wait_loads<0>();
      } else {
        wait_loads_at_most<kPieces * (kStages - 2 > 0 ? kStages - 2 : 0)>(pieces_a_tile * min(kStages - 2, kt_end - 1 - kt));
      }
      lds_barrier();
      if (kt + kStages - 1 < kt_end) stage_ask(kt + kStages - 1, (kt - kt_begin + kStages - 1) % kStages);
#pragma unroll
      for (int h = 0; h < 2; ++h) cur.ok[h] = kt * 32 + 16 * h <= walk_max && kt * 32 + 16 * h + 15 >= lo_min;
      if (kt < own_first || kt > own_last) continue;      // no key of this wave's rows in the tile
    } else if constexpr (kAhead) {
      if (kt + 1 < kt_end) fetch(nxt, kt + 1);
    } else {
      fetch(cur, kt);
    }
    const int key0 = kt * 32;
    // values of keys past the walk's last position may never have been written: they are replaced
    // by zero (in the tile at the end only)
    const bool edge = key0 + 31 > walk_max;
    auto value_fragment = [&](int b) -> uint4 {
      uint2 v0, v1;
      if constexpr (kStaged) {
        v0 = *reinterpret_cast<const uint2*>(tile_lds + 32 * d + 256 * b + v_lane);
        v1 = *reinterpret_cast<const uint2*>(tile_lds + 48 * d + 256 * b + v_lane);
      } else {
        v0 = cur.v[0][b];
        v1 = cur.v[1][b];
      }
      if (edge) {
        int kb = key0 + 4 * grp;
        // (pinned here: left alone, the compiler works the masks out in every tile, before the branch)
        asm volatile("" : "+v"(kb));
        v0.x &= (kb <= walk_max ? 0xffffu : 0u) | (kb + 1 <= walk_max ? 0xffff0000u : 0u);
        v0.y &= (kb + 2 <= walk_max ? 0xffffu : 0u) | (kb + 3 <= walk_max ? 0xffff0000u : 0u);
        v1.x &= (kb + 16 <= walk_max ? 0xffffu : 0u) | (kb + 17 <= walk_max ? 0xffff0000u : 0u);
        v1.y &= (kb + 18 <= walk_max ? 0xffffu : 0u) | (kb + 19 <= walk_max ? 0xffff0000u : 0u);
      }
      return make_uint4(v0.x, v0.y, v1.x, v1.y);
    };
    auto key_fragment = [&](int h, int j) -> uint4 {
      if constexpr (kStaged) {
        return (EXACT || 32 * j + 8 * grp < d) ? *reinterpret_cast<const uint4*>(tile_lds + 16 * d * h + 512 * j + k_lane)
                                               : zero16();
      } else {
        return cur.k[h][j];
      }
    };
    // The wave's query tiles go through each phase together -- all score MFMAs, then all the
    // softmax arithmetic, then all output MFMAs -- with no branch between tiles, so that the
    // independent chains of the tiles overlap.  (Tiles beyond the request's rows run masked.)
    floatx4 sc[QT][2];
#pragma unroll
    for (int t = 0; t < QT; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) sc[t][h] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int j = 0; j < DJ; ++j) {
        const uint4 kf = key_fragment(h, j);
#pragma unroll
        for (int t = 0; t < QT; ++t) sc[t][h] = mfma_16x16x32(kf, qf[t][j], sc[t][h]);
      }
    // A lane holds, for its query row, the raw scores of keys key0 + 16h + 4*grp + r.  A key tile
    // that every row of the wave sees whole needs no mask (the usual case away from the diagonal);
    // otherwise scores are masked by position, window and row validity.
    const int last_lo = (a.window > 0 && pos_max - a.window + 1 > 0) ? pos_max - a.window + 1 : 0;
    const bool interior = key0 + 31 <= pos_min && key0 >= last_lo && ntok == a.tpt * QT;
    float sv[QT][8];
    if (interior) {
#pragma unroll
      for (int t = 0; t < QT; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r) sv[t][4 * h + r] = sc[t][h][r];
    } else {
#pragma unroll
      for (int t = 0; t < QT; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int key = key0 + 16 * h + 4 * grp + r;
            const bool vis = cur.ok[h] && q_ok[t] && key <= q_pos[t] && key >= q_lo[t];
            sv[t][4 * h + r] = vis ? sc[t][h][r] : -INFINITY;
          }
    }
    // The exponents are taken against a reference per row, kept over raw scores (the softmax scale, > 0,
    // enters the exponent): a maximum the row has seen, moved up to the tile's maximum only when that
    // exceeds it by more than kSlack in the exponent.  Probabilities then reach 2^kSlack at most, which
    // float sums and bfloat16 factors hold as well as values up to 1, and the quotient of the two sums
    // does not depend on the reference -- but what has been summed is scaled down far less often (with
    // the latest maximum as reference some row of a wave's 64 moves in most of a prompt's tiles).
    // A lane first looks at its own eight scores only: while none of the wave's lanes sees one beyond its row's
    // reference by more than the slack -- every tile but a walk's first few -- the rows' maxima need not be
    // found across lanes, nothing moves, and the exponents' shift is the one kept from before.
    constexpr float kSlack = 8.0f;
    float lane_max[QT];
    bool beyond = false;
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float m_lane = max3(sv[t][0], sv[t][1], sv[t][2]);
      m_lane = max3(m_lane, sv[t][3], sv[t][4]);
      m_lane = max3(m_lane, sv[t][5], sv[t][6]);
      lane_max[t] = max2(m_lane, sv[t][7]);
      beyond = beyond || lane_max[t] > m_limit[t];                     // (from -inf: any score is)
    }
    if (__any(beyond)) {
      // Some row of the wave may have to move its reference (early in a walk, rarely later): the rows' maxima
      // are found, and what has been summed so far is scaled down by 2^(old reference - new reference), 0 while
      // nothing had been seen.
#pragma unroll
      for (int t = 0; t < QT; ++t) {
        const float m_tile = max_16_32(lane_max[t]);
        const bool up = (m_tile - m_run[t]) * a.scale_log2 > kSlack;   // (from -inf: yes; nothing seen in the tile: no)
        const float m_new = up ? m_tile : m_run[t];
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2((m_run[t] - m_safe) * a.scale_log2);
        l_run[t] *= alpha;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[t][b][r] *= alpha;
        m_run[t] = m_new;
        m_shift[t] = -m_safe * a.scale_log2;
        m_limit[t] = m_new + kSlack / a.scale_log2;                    // (-inf stays -inf)
      }
    }
    uint4 pf[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      float p[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = fast_exp2(fmaf(sv[t][i], a.scale_log2, m_shift[t]));
      l_run[t] += ((p[0] + p[1]) + (p[2] + p[3])) + ((p[4] + p[5]) + (p[6] + p[7]));
      pf[t] = make_uint4(pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                         pack_bf16x2(p[6], p[7]));
    }
    // (blocks past the head size hold zeros and are never stored)
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      const uint4 vf = value_fragment(b);
#pragma unroll
      for (int t = 0; t < QT; ++t) o[t][b] = mfma_16x16x32(vf, pf[t], o[t][b]);
    }
    if constexpr (kAhead && !kStaged) {
      if (kt + 1 < kt_end) cur = nxt;
    }
  }

  if constexpr (WS > 1) {
    // The waves' partial results meet in LDS; then all threads share out the tile's 16 x d
    // outputs and add the parts in wave order, weighted by 2^(m_part - m).
    const int ostride = d + kMergePad;
    float* part_o = merge_raw;
    float* part_ml = merge_raw + WS * 16 * ostride;
    const float l_tot = sum_16_32(l_run[0]);
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      if (!EXACT && 16 * b >= d) break;
      *reinterpret_cast<floatx4*>(part_o + (wave * 16 + col) * ostride + 16 * b + 4 * grp) = o[0][b];
    }
    if (grp == 0) {
      part_ml[(wave * 16 + col) * 2] = m_run[0] * a.scale_log2;      // (-inf stays -inf: the scale is > 0)
      part_ml[(wave * 16 + col) * 2 + 1] = l_tot;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < 16 * d; idx += WS * kWave) {
      const int r = idx / d, c = idx % d;
      const int r_tok = r / a.hg, r_head_in_group = hsub * a.hg + r % a.hg;
      if (r_tok >= a.tpt || r_tok >= ntok || r_head_in_group >= group) continue;
      float m = -INFINITY;
#pragma unroll
      for (int w = 0; w < WS; ++w) m = fmaxf(m, part_ml[(w * 16 + r) * 2]);
      float l = 0.f, acc = 0.f;
#pragma unroll
      for (int w = 0; w < WS; ++w) {
        const float mw = part_ml[(w * 16 + r) * 2];
        const float wt = (mw == -INFINITY) ? 0.f : fast_exp2(mw - m);
        l += wt * part_ml[(w * 16 + r) * 2 + 1];
        acc += wt * part_o[(w * 16 + r) * ostride + c];
      }
      const long row = row0 + tok0 + r_tok;
      const int head = kvh * group + r_head_in_group;
      if (a.n_splits == 1) {
        a.out[(row * a.n_heads + head) * d + c] = from_float<bf16_t>(acc / l);
      } else {
        const long slot = (static_cast<long>(part) * a.n_tokens + row) * a.n_heads + head;
        a.part_o[slot * d + c] = acc;
        if (c == 0) {
          a.part_ml[slot * 2] = m;
          a.part_ml[slot * 2 + 1] = l;
        }
      }
    }
    return;
  }

#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const float l_tot = sum_16_32(l_run[t]);
    if (!q_ok[t]) continue;
    const long row = row0 + tok0 + q_tok[t];
    if (a.n_splits == 1 || (listed && n_parts == 1)) {      // (a walk that was not cut: nothing to merge)
      const float inv = 1.0f / l_tot;
      bf16_t* dst = a.out + (row * a.n_heads + q_head) * d + 4 * grp;
#pragma unroll
      for (int b = 0; b < DB; ++b) {
        if (!EXACT && 16 * b >= d) break;
        uint2 pack;
        pack.x = pack_bf16x2(o[t][b][0] * inv, o[t][b][1] * inv);
        pack.y = pack_bf16x2(o[t][b][2] * inv, o[t][b][3] * inv);
        *reinterpret_cast<uint2*>(dst + 16 * b) = pack;
      }
    } else {
      const long slot = (static_cast<long>(part) * a.n_tokens + row) * a.n_heads + q_head;
      float* dst = a.part_o + slot * d + 4 * grp;
#pragma unroll
      for (int b = 0; b < DB; ++b) {
        if (!EXACT && 16 * b >= d) break;
        *reinterpret_cast<floatx4*>(dst + 16 * b) = o[t][b];
      }
      if (grp == 0) {
        a.part_ml[slot * 2] = m_run[t] * a.scale_log2;
        a.part_ml[slot * 2 + 1] = l_tot;
      }
    }
  }
}

// out[row, head, :] = sum_z 2^(m_z - M) O_z / sum_z 2^(m_z - M) l_z, parts added in order of z.
// One wave per (row, head), up to 64 parts: lane z reads part z's statistics, the weights go
// through LDS, and every lane then sums its output dimensions over the parts.  With row_seq given,
// rows of requests that had no tile in this launch (tile_start[s + 1] == tile_start[s]) are left
// alone: another launch writes them.
constexpr int kMaxSplits = 64;

__global__ __launch_bounds__(kWave) void attention_merge_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                bf16_t* __restrict__ out, int n_splits,
                                                                long n_rows_heads, int d, int n_heads,
                                                                const int32_t* __restrict__ row_seq,
                                                                const int32_t* __restrict__ tile_start) {
  __shared__ float weight[kMaxSplits];
  const long rh = blockIdx.x;
  const int lane = threadIdx.x;
  if (row_seq != nullptr) {
    const int s = row_seq[rh / n_heads];
    if (tile_start[s + 1] == tile_start[s]) return;
  }
  // the first parts' outputs are asked for together with the statistics, not after them
  constexpr int kEarly = 8;
  float early[kEarly];
#pragma unroll
  for (int z = 0; z < kEarly; ++z) early[z] = (z < n_splits && lane < d) ? part_o[(z * n_rows_heads + rh) * d + lane] : 0.f;
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
    int z = 0;
    if (c == lane) {
#pragma unroll
      for (; z < kEarly; ++z) acc += weight[z] * early[z];      // (weights beyond n_splits are zero)
    }
#pragma unroll 8
    for (; z < n_splits; ++z) acc += weight[z] * part_o[(z * n_rows_heads + rh) * d + c];
    out[rh * d + c] = from_float<bf16_t>(acc * inv);
  }
}

// The same for up to MAXS parts (the usual case: prompts are cut into at most 8, decode steps of
// short contexts into few): a thread takes four neighbouring output dimensions of one (row, head),
// asks for every part's statistics and outputs at once -- one trip to memory, no LDS, no barrier --
// and adds the parts in order of z.
// row_parts (with a work list): how many parts row t's keys were cut into; a row with one part has been
// written by the attention kernel and is left alone.
template <int MAXS>
__global__ __launch_bounds__(256) void attention_merge_few_kernel(const float* __restrict__ part_o,
                                                                  const float* __restrict__ part_ml,
                                                                  bf16_t* __restrict__ out, int n_splits,
                                                                  long n_rows_heads, int d, int n_heads,
                                                                  const int32_t* __restrict__ row_seq,
                                                                  const int32_t* __restrict__ tile_start,
                                                                  const int32_t* __restrict__ row_parts) {
  const long item = blockIdx.x * 256L + threadIdx.x;
  const int per = d / 4;
  const long rh = item / per;
  const int c = static_cast<int>(item % per) * 4;
  if (rh >= n_rows_heads) return;
  if (row_seq != nullptr) {
    const int s = row_seq[rh / n_heads];
    if (tile_start[s + 1] == tile_start[s]) return;
  }
  if (row_parts != nullptr) {
    n_splits = row_parts[rh / n_heads];
    if (n_splits <= 1) return;
  }
  float2 ml[MAXS];
  floatx4 o[MAXS];
#pragma unroll
  for (int z = 0; z < MAXS; ++z) {
    const bool live = z < n_splits;
    ml[z] = live ? *reinterpret_cast<const float2*>(part_ml + (z * n_rows_heads + rh) * 2) : make_float2(-INFINITY, 0.f);
    o[z] = live ? *reinterpret_cast<const floatx4*>(part_o + (z * n_rows_heads + rh) * d + c) : floatx4{0.f, 0.f, 0.f, 0.f};
  }
  float m = -INFINITY;
#pragma unroll
  for (int z = 0; z < MAXS; ++z) m = fmaxf(m, ml[z].x);
  float l = 0.f;
  floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int z = 0; z < MAXS; ++z) {
    const float wz = (ml[z].x == -INFINITY) ? 0.f : exp2f(ml[z].x - m);
    l += wz * ml[z].y;
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] += wz * o[z][e];
  }
  const float inv = 1.0f / l;
  uint2 pack;
  pack.x = pack_bf16x2(acc[0] * inv, acc[1] * inv);
  pack.y = pack_bf16x2(acc[2] * inv, acc[3] * inv);
  *reinterpret_cast<uint2*>(out + rh * d + c) = pack;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

namespace bc4g {
namespace {
template <int DJ, int DB, int QT, int WS>
int launch_attention(const AttnArgs& a, dim3 grid, dim3 block, size_t lds, hipStream_t s) {
  // per instantiation, once: the staged form's ring may need more than the default dynamic LDS
  static std::once_flag once;
  static hipError_t raised = hipSuccess;
  if (lds > 48 * 1024) {
    std::call_once(once, [] {
      raised = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_mfma_kernel<DJ, DB, QT, WS, true>),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (raised == hipSuccess)
        raised = hipFuncSetAttribute(reinterpret_cast<const void*>(attention_mfma_kernel<DJ, DB, QT, WS, false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    });
    if (raised != hipSuccess)
      return fail("attention_mfma: cannot raise the dynamic LDS limit to the %zu bytes of the key tiles' ring (%s)", lds,
                  hipGetErrorString(raised));
  }
  if (a.head_dim == 16 * DB) attention_mfma_kernel<DJ, DB, QT, WS, true><<<grid, block, lds, s>>>(a);
  else attention_mfma_kernel<DJ, DB, QT, WS, false><<<grid, block, lds, s>>>(a);
  return 0;
}
}  // namespace
}  // namespace bc4g

extern "C" int bc4g_attention_mfma(const void* qkv, int q_stride, void* out, float* part_o, float* part_ml, const void* k_cache,
                                   const void* v_cache, const int32_t* block_table, int table_stride,
                                   const int32_t* seq_start, const int32_t* seq_ctx, const int32_t* tile_start,
                                   int n_seqs, int n_tiles, int n_tokens, int n_heads, int n_kv_heads, int head_dim,
                                   int page_tokens, int window, float scale, int tokens_per_tile, int q_tiles,
                                   int form, int n_splits, const int32_t* items, int n_items, const int32_t* row_parts,
                                   int single_rows, const int32_t* row_seq, void* stream) {
  BC4G_REQUIRE(n_heads > 0 && n_kv_heads > 0 && n_heads % n_kv_heads == 0, "attention_mfma: bad heads %d/%d",
               n_heads, n_kv_heads);
  BC4G_REQUIRE(head_dim >= 16 && head_dim <= 256 && head_dim % 16 == 0,
               "attention_mfma: head_dim %d must be a multiple of 16 up to 256", head_dim);
  BC4G_REQUIRE(page_tokens > 0 && page_tokens % 16 == 0, "attention_mfma: page_tokens %d must be a multiple of 16",
               page_tokens);
  BC4G_REQUIRE(n_splits >= 1 && n_splits <= kMaxSplits && (n_splits == 1 || (part_o && part_ml)),
               "attention_mfma: the split count %d must lie in 1..64", n_splits);
  BC4G_REQUIRE(window >= 0 && table_stride > 0 && n_seqs > 0, "attention_mfma: bad sizes");
  BC4G_REQUIRE(items == nullptr || (form == 2 && row_parts != nullptr && n_items > 0 && n_items <= 65535 && n_splits <= 8 &&
                                    n_tiles < (1 << 20)),
               "attention_mfma: a work list goes with the staged prompt form, the rows' part counts, at most 65535 items, "
               "8 parts and 2^20 pieces (form %d, %d items, %d parts, %d pieces)", form, n_items, n_splits, n_tiles);
  BC4G_REQUIRE(scale > 0.f, "attention_mfma: the softmax scale must be positive, got %g", static_cast<double>(scale));
  BC4G_REQUIRE(q_stride >= n_heads * head_dim && q_stride % 8 == 0, "attention_mfma: bad query row stride %d", q_stride);
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
  a.q_stride = q_stride;
  a.n_heads = n_heads;
  a.n_kv_heads = n_kv_heads;
  a.head_dim = head_dim;
  a.page_tokens = page_tokens;
  a.window = window;
  a.hg = group < 16 ? group : 16;
  a.tpt = tokens_per_tile;
  a.n_sub = (group + a.hg - 1) / a.hg;
  a.n_splits = n_splits;
  a.items = items;
  a.row_parts = items ? row_parts : nullptr;
  a.single_rows = single_rows ? 1 : 0;
  BC4G_REQUIRE(!single_rows || (form == 1 && n_tiles == n_seqs && n_tokens == n_seqs),
               "attention_mfma: single rows means one row and one tile a request in the decode form (%d requests, %d "
               "tiles, %d rows)", n_seqs, n_tiles, n_tokens);
  a.scale_log2 = scale * kLog2e;
  BC4G_REQUIRE(a.tpt >= 1 && a.tpt * a.hg <= 16, "attention_mfma: %d tokens x %d heads do not fit a 16-row tile",
               a.tpt, a.hg);
  const int dj = (head_dim + 31) / 32, db = head_dim / 16;
  const int max_qt = db <= 4 ? 4 : (db <= 8 ? 2 : 1);
  BC4G_REQUIRE(q_tiles == 1 || (q_tiles == max_qt && (q_tiles == 2 || q_tiles == 4)),
               "attention_mfma: %d query tiles per wave are not built for head_dim %d (1 or %d)", q_tiles, head_dim,
               max_qt);
  BC4G_REQUIRE(n_kv_heads * a.n_sub <= 65535, "attention_mfma: too many heads for the grid");
  BC4G_REQUIRE(form >= 0 && form <= 2, "attention_mfma: unknown form %d", form);
  BC4G_REQUIRE(form != 1 || q_tiles == 1, "attention_mfma: waves share the keys of single query tiles only");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int status = 0;
  if (form == 2) {
    // four waves' tiles per workgroup (n_tiles counts workgroups), key tiles staged in a ring in LDS
    // (with a work list: heads fastest, so that the items start in the list's order, longest first)
    dim3 grid(n_tiles, n_kv_heads * a.n_sub, n_splits);
    if (items) grid = dim3(n_kv_heads * a.n_sub, n_items, 1);
    dim3 block(kWavesPerBlock * kWave);
    const size_t lds = static_cast<size_t>(db <= 8 ? 4 : 2) * 128 * head_dim + 1024 * 4;   // (the kernel's ring of key tiles and its part of the block table)
    if (dj <= 2 && db <= 4) {
      if (q_tiles == 4) status = launch_attention<2, 4, 4, 0>(a, grid, block, lds, s);
      else status = launch_attention<2, 4, 1, 0>(a, grid, block, lds, s);
    } else if (dj <= 4 && db <= 8) {
      if (q_tiles == 2) status = launch_attention<4, 8, 2, 0>(a, grid, block, lds, s);
      else status = launch_attention<4, 8, 1, 0>(a, grid, block, lds, s);
    } else {
      status = launch_attention<8, 16, 1, 0>(a, grid, block, lds, s);
    }
  } else if (form == 1) {
    // one workgroup per tile; its waves (8, or 4 for the largest heads) cut the keys between them
    dim3 grid(n_tiles, n_kv_heads * a.n_sub, n_splits);
    auto lds = [&](int ws) { return static_cast<size_t>(ws) * 16 * (head_dim + kMergePad + 2) * sizeof(float); };
    if (dj <= 2 && db <= 4) status = launch_attention<2, 4, 1, 8>(a, grid, 8 * kWave, lds(8), s);
    else if (dj <= 4 && db <= 8) status = launch_attention<4, 8, 1, 8>(a, grid, 8 * kWave, lds(8), s);
    else status = launch_attention<8, 16, 1, 4>(a, grid, 4 * kWave, lds(4), s);
  } else {
    dim3 grid((n_tiles + kWavesPerBlock - 1) / kWavesPerBlock, n_kv_heads * a.n_sub, n_splits);
    dim3 block(kWavesPerBlock * kWave);
    if (dj <= 2 && db <= 4) {
      if (q_tiles == 4) status = launch_attention<2, 4, 4, 1>(a, grid, block, 0, s);
      else status = launch_attention<2, 4, 1, 1>(a, grid, block, 0, s);
    } else if (dj <= 4 && db <= 8) {
      if (q_tiles == 2) status = launch_attention<4, 8, 2, 1>(a, grid, block, 0, s);
      else status = launch_attention<4, 8, 1, 1>(a, grid, block, 0, s);
    } else {
      status = launch_attention<8, 16, 1, 1>(a, grid, block, 0, s);
    }
  }
  if (status) return status;
  if (int e = check_launch("attention_mfma")) return e;
  if (n_splits > 1) {
    const long rows_heads = static_cast<long>(n_tokens) * n_heads;
    BC4G_REQUIRE(rows_heads <= 2147483647L, "attention_mfma: too many rows to merge");
    constexpr int kFew = 8;
    if (n_splits <= kFew) {
      const long work = rows_heads * (head_dim / 4);
      attention_merge_few_kernel<kFew><<<static_cast<unsigned>((work + 255) / 256), 256, 0, s>>>(
          part_o, part_ml, a.out, n_splits, rows_heads, head_dim, n_heads, row_seq, tile_start, a.row_parts);
    } else {
      attention_merge_kernel<<<static_cast<unsigned>(rows_heads), 64, 0, s>>>(part_o, part_ml, a.out, n_splits,
                                                                               rows_heads, head_dim, n_heads, row_seq,
                                                                               tile_start);
    }
    return check_launch("attention_merge");
  }
  return 0;
}
