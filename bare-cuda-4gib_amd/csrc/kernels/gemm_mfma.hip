// out[m, n] (+)= sum_k a[m, k] * w[n, k], bfloat16 operands, float accumulation on the matrix
// cores: the product of prompt portions (many rows).
//
// A workgroup of 4 waves computes a 128 x 128 tile of the output in k-steps of 64.  Both operands
// are contiguous in k, so a tile of each is staged through LDS as [128 rows][64 k] with rows padded
// to 144 bytes (which makes the 16-byte fragment reads of 8 consecutive lanes cover all banks), in
// two buffers: while the waves feed 32x32x16 MFMAs from one, the next k-step is written to the other
// and the two after it are in flight from memory, in registers.  Each wave owns a 64 x 64 quarter
// (2 x 2 MFMA blocks).  The finished tile leaves through LDS in 16-byte pieces.
// Rows and columns beyond the matrix are read as zero and not stored; k must be a multiple of 8.
// Every output element is accumulated over k in ascending order, whatever the number of rows.
//
// What bounds this kernel is not the matrix cores but what a CU can pull through its cache: at
// 128 x 128 a k-step of 64 brings 32 KB for 2 MFLOP, and 256 CUs doing so reach ~10 TB/s together
// (measured: ~650 TFLOP/s).  Where the output has tiles enough, a workgroup of 8 waves therefore
// takes a 256 x 128 tile (the same waves a CU, the same per-wave work, a quarter less traffic).
//
// Workgroups are numbered so that those sharing tiles of a and w run on the same XCD at the same
// time (tile_of).  Where 256 x 256 tiles fill the CUs, a third form takes those (gemm_mfma_wide_kernel).
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kBM = 128, kBN = 128, kBK = 64;
constexpr int kLdsStride = kBK + 8;   // elements; 144 bytes
constexpr int kXcds = 8;

// kSwigluBf16: every 16 rows of w are eight gate rows and the eight up rows of the same outputs;
// out [m, n / 2] = silu(gate) * up.  A gate and its up lie eight lanes apart in the MFMA result.
enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAccumF32 = 2, kSwigluBf16 = 3 };


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

struct Tile {
  bf16_t a[kBM][kLdsStride];
  bf16_t w[kBN][kLdsStride];
};

// Stores a finished tile (float [128][kBN + 4] in LDS) with the epilogue, THREADS threads together.
template <int EPI, int THREADS>
__device__ inline void store_tile(const float* tile_out, void* __restrict__ out, int m, int n, long m0, long n0, int tid) {
  constexpr int kOutStride = kBN + 4;
  const bool vec = n % 4 == 0;      // rows of the output start on 16-byte (bfloat16: 8-byte) boundaries
  if constexpr (EPI == kSwigluBf16) {
    // every 16 columns: eight gates, then the eight ups of the same outputs; a thread takes four gates
    const long n_out = n / 2;
    for (int c = tid; c < kBM * (kBN / 8); c += THREADS) {
      const int row = c / (kBN / 8), q = c % (kBN / 8);           // q: group of four outputs
      const int col = (q / 2) * 16 + (q % 2) * 4;                 // first gate column in the tile
      const long gm = m0 + row, gn = n0 + col;
      if (gm >= m || gn >= n) continue;
      const float* src = tile_out + row * kOutStride + col;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (src[e] / (1.0f + expf(-src[e]))) * src[e + 8];
      bf16_t* dst = static_cast<bf16_t*>(out) + gm * n_out + (gn / 16) * 8 + gn % 16;
      if (n_out % 4 == 0) {
        uint2 pk;
        pk.x = static_cast<uint32_t>(bf16_bits_from_float(v[0])) | (static_cast<uint32_t>(bf16_bits_from_float(v[1])) << 16);
        pk.y = static_cast<uint32_t>(bf16_bits_from_float(v[2])) | (static_cast<uint32_t>(bf16_bits_from_float(v[3])) << 16);
        *reinterpret_cast<uint2*>(dst) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) dst[e] = from_float<bf16_t>(v[e]);
      }
    }
  } else {
    for (int c = tid; c < kBM * (kBN / 4); c += THREADS) {
      const int row = c / (kBN / 4), col = (c % (kBN / 4)) * 4;
      const long gm = m0 + row, gn = n0 + col;
      if (gm >= m || gn >= n) continue;
      const floatx4 v = *reinterpret_cast<const floatx4*>(tile_out + row * kOutStride + col);
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

// SETS: register sets; SETS - 1 k-steps are in flight from memory while one is written to LDS.
// WMS: rows of waves (64 output rows each) -- 2 for the 128 x 128 tile, 4 for the 256 x 128 one.
template <int WMS>
struct TileOf {
  bf16_t a[64 * WMS][kLdsStride];
  bf16_t w[kBN][kLdsStride];
};

template <int EPI, int SETS, int WMS>
__global__ __launch_bounds__(128 * WMS, WMS == 2 ? 2 : 1) void gemm_mfma_kernel(
    const bf16_t* __restrict__ a, const bf16_t* __restrict__ w, void* __restrict__ out, int m, int n, int k,
    int m_blocks, int n_blocks) {
  constexpr int kRows = 64 * WMS, kThreads = 128 * WMS;
  constexpr int kChunkRows = kThreads / 8;           // rows one chunk of a thread's loads covers
  constexpr int kChunksA = kRows / kChunkRows, kChunksW = kBN / kChunkRows;
  typedef TileOf<WMS> Tile;
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

  // The tile goes out through LDS (as float [128][128 + 4], 128 rows at a time), so that a thread
  // stores four neighbouring columns of a row at once.  acc[i][j][r] is row wm*64 + i*32 + 8*(r/4) +
  // 4*(lane/32) + r%4 and column wn*64 + j*32 + lane%32 of the tile.
  constexpr int kOutStride = kBN + 4;
  static_assert(sizeof(float) * kBM * kOutStride <= sizeof(Tile) * 2, "the output tile must fit the operand buffers");
  float* tile_out = reinterpret_cast<float*>(lds_raw);
#pragma unroll
  for (int half = 0; half < WMS / 2; ++half) {
    if (half > 0) lds_barrier();                      // the half before has been read
    if (wm / 2 == half) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            tile_out[((wm % 2) * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4) * kOutStride + wn * 64 + j * 32 +
                     lane % 32] = acc[i][j][r];
    }
    lds_barrier();
    store_tile<EPI, kThreads>(tile_out, out, m, n, m0 + 128 * half, n0, tid);
  }
}

// The same product with the work split between waves: four waves only multiply, eight only move
// operands (memory -> registers -> LDS).  A wave issues its instructions in order, so a wave that
// does everything stands still at a full memory queue with its MFMAs behind it; here the
// multiplying waves wait for data only.  The moving waves form two groups that take the k-steps in
// turn: in a round one group writes its step into LDS while the other asks memory for a later one
// -- writing a step takes about as long as asking for one (measured: 900 and 1,300 clocks for a
// 48 KB step), and one group doing both in a row was what a round waited for.  LDS holds three
// k-steps: while step t is multiplied, step t + 2 is written; each group has two more in flight
// in registers.
constexpr int kStages = 3, kSets = 2;
constexpr int kSplitThreads = 768;

template <int EPI>
__global__ __launch_bounds__(kSplitThreads) void gemm_mfma_split_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                              void* __restrict__ out, int m, int n, int k,
                                                              int m_blocks, int n_blocks) {
  __shared__ __align__(16) unsigned char lds_raw[sizeof(Tile) * kStages];
  Tile* tiles = reinterpret_cast<Tile*>(lds_raw);
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const bool mover = wave >= 4;

  int bm, bn;
  tile_of(blockIdx.x, m_blocks, n_blocks, bm, bn);
  const long m0 = static_cast<long>(bm) * kBM, n0 = static_cast<long>(bn) * kBN;
  const int nk = (k + kBK - 1) / kBK;

  floatx16 acc[2][2];
  const int wm = (wave % 4) / 2, wn = wave % 2;   // a multiplying wave's 64 x 64 quarter

  if (mover) {
    // thread u of a group's 256 takes segment u % 8 of rows u / 8 + 32 i of both operands
    const int group = (wave - 4) / 4;             // owns the k-steps s with s % 2 == group
    const int u = tid - 256 - 256 * group, seg = u % 8, lrow = u / 8;
    struct Staged {
      uint4 a[4], w[4];
    };
    const bf16_t* arow[4];
    const bf16_t* wrow[4];
    bool a_ok[4], w_ok[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const long gm = m0 + lrow + 32 * i, gn = n0 + lrow + 32 * i;
      a_ok[i] = gm < m;
      w_ok[i] = gn < n;
      arow[i] = a + (a_ok[i] ? gm : 0) * k + seg * 8;
      wrow[i] = w + (w_ok[i] ? gn : 0) * k + seg * 8;
    }
    auto load_step = [&](Staged& r, int kt) {
      const int kk = kt * kBK;
      const bool k_ok = kk + seg * 8 < k;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        r.a[i] = (k_ok && a_ok[i]) ? load16(arow[i] + kk) : zero16();
        r.w[i] = (k_ok && w_ok[i]) ? load16(wrow[i] + kk) : zero16();
      }
    };
    auto store_step = [&](const Staged& r, int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *reinterpret_cast<uint4*>(&tiles[buf].a[lrow + 32 * i][seg * 8]) = r.a[i];
        *reinterpret_cast<uint4*>(&tiles[buf].w[lrow + 32 * i][seg * 8]) = r.w[i];
      }
    };
    // Step s lands in LDS buffer s % kStages; steps 0 and 1 before the first round, step t + 2 in
    // round t.  A group's step s >= 2 travels in its register set (s / 2 - 1) % kSets.  In round t
    // the group of step t + 2 (t % 2) stores it; the other group asks for step t + 1 + 2 kSets into
    // the set its step t + 1 left the round before.
    Staged r[kSets];
    if (group < nk) {
      load_step(r[0], group);
      store_step(r[0], group);
    }
#pragma unroll
    for (int i = 0; i < kSets; ++i)
      if (2 + group + 2 * i < nk) load_step(r[i], 2 + group + 2 * i);
    lds_barrier();
    constexpr int kUnroll = 12;   // lcm(kStages, 2 groups x kSets)
    for (int kt = 0; kt < nk; kt += kUnroll) {
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) {
        const int t = kt + j;
        if (t >= nk) break;
        if (group == j % 2) {
          if (t + 2 < nk) store_step(r[(j / 2) % kSets], (j + 2) % kStages);
        } else if (t >= 1) {
          if (t + 1 + 2 * kSets < nk) load_step(r[((j + 1) / 2 + kSets - 1) % kSets], t + 1 + 2 * kSets);
        }
        lds_barrier();
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    const int frow = lane % 32, fk = (lane / 32) * 8;
    lds_barrier();
    constexpr int kUnroll = 3;
    for (int kt = 0; kt < nk; kt += kUnroll) {
#pragma unroll
      for (int j = 0; j < kUnroll; ++j) {
        const int t = kt + j;
        if (t >= nk) break;
        const int cur = j % kStages;
#pragma unroll
        for (int ks = 0; ks < kBK / 16; ++ks) {
          uint4 fa[2], fw[2];
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            fa[i] = *reinterpret_cast<const uint4*>(&tiles[cur].a[wm * 64 + i * 32 + frow][ks * 16 + fk]);
            fw[i] = *reinterpret_cast<const uint4*>(&tiles[cur].w[wn * 64 + i * 32 + frow][ks * 16 + fk]);
          }
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) acc[i][jj] = mfma_32x32x16(fa[i], fw[jj], acc[i][jj]);
        }
        lds_barrier();
      }
    }
  }

  // The tile goes out through LDS (as float [128][128 + 4]): all threads store it, four
  // neighbouring columns of a row at once.
  constexpr int kOutStride = kBN + 4;
  float* tile_out = reinterpret_cast<float*>(lds_raw);
  if (!mover) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          tile_out[(wm * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4) * kOutStride + wn * 64 + j * 32 + lane % 32] =
              acc[i][j][r];
  }
  lds_barrier();
  store_tile<EPI, kSplitThreads>(tile_out, out, m, n, m0, n0, tid);
}

// The same product for outputs with very many tiles: a workgroup of 8 waves takes a 256 x 256 tile
// and a wave a 128 x 64 part of it (4 x 2 MFMA blocks).  Per FLOP the tile brings two thirds of the
// bytes of a 256 x 128 one through the CU's cache, which is what bounds these kernels, and a wave
// reads three quarters of the fragments from LDS (measured, with the banded tile order:
// 4096 x 4096 x 4096 833 -> 1,015 TFLOP/s, 8192 x 6144 x 4096 917 -> 1,044; no gain where k is long
// and the output wide, 8192 x 28672 x 4096).  A k-step of 64 is 72 KB in LDS, in two buffers; the
// step after the next is in flight in registers: between the MFMAs of each slice of 16 a quarter of it
// is written to LDS and asked for again, two steps ahead, and the next slice's fragments are read
// while this slice's MFMAs run.  The order of the additions over k is that of the other forms.
constexpr int kWide = 256;
struct WideTile {
  bf16_t a[kWide][kLdsStride];
  bf16_t w[kWide][kLdsStride];
};
constexpr size_t kWideLdsBytes = sizeof(WideTile) * 2;

template <int EPI>
__global__ __launch_bounds__(512, 1) void gemm_mfma_wide_kernel(const bf16_t* __restrict__ a, const bf16_t* __restrict__ w,
                                                                     void* __restrict__ out, int m, int n, int k,
                                                                     int m_blocks, int n_blocks) {
  constexpr int WN = 4;                         // waves along n (two rows of them along m)
  constexpr int kThreads = 128 * WN;
  constexpr int kWaveN = kWide / WN;            // columns of a wave's part
  constexpr int kJ = kWaveN / 32;               // MFMA blocks along n
  extern __shared__ __align__(16) unsigned char wide_raw[];
  WideTile* tiles = reinterpret_cast<WideTile*>(wide_raw);
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave / WN, wn = wave % WN;

  int bm, bn;
  tile_of(blockIdx.x, m_blocks, n_blocks, bm, bn);
  const long m0 = static_cast<long>(bm) * kWide, n0 = static_cast<long>(bn) * kWide;

  // global -> LDS: thread t moves segment t % 8 (16 bytes) of rows t / 8 + kChunkRows i of both operands
  constexpr int kChunkRows = kThreads / 8;
  constexpr int kChunks = kWide / kChunkRows;
  constexpr int kPerSlice = kChunks / (kBK / 16);   // chunks written and asked for again per slice of k
  static_assert(kPerSlice >= 1, "a slice moves at least one chunk");
  const int seg = tid % 8, lrow = tid / 8;
  uint4 ra[kChunks], rw[kChunks];
  const bf16_t* arow[kChunks];
  const bf16_t* wrow[kChunks];
  bool a_ok[kChunks], w_ok[kChunks];
#pragma unroll
  for (int i = 0; i < kChunks; ++i) {
    const long gm = m0 + lrow + kChunkRows * i, gn = n0 + lrow + kChunkRows * i;
    a_ok[i] = gm < m;
    w_ok[i] = gn < n;
    arow[i] = a + (a_ok[i] ? gm : 0) * k + seg * 8;
    wrow[i] = w + (w_ok[i] ? gn : 0) * k + seg * 8;
  }
  auto load_chunk = [&](int kt, int i) {
    const int kk = kt * kBK;
    const bool k_ok = kk + seg * 8 < k;
    ra[i] = (k_ok && a_ok[i]) ? load16(arow[i] + kk) : zero16();
    rw[i] = (k_ok && w_ok[i]) ? load16(wrow[i] + kk) : zero16();
  };
  auto store_chunk = [&](int buf, int i) {
    *reinterpret_cast<uint4*>(&tiles[buf].a[lrow + kChunkRows * i][seg * 8]) = ra[i];
    *reinterpret_cast<uint4*>(&tiles[buf].w[lrow + kChunkRows * i][seg * 8]) = rw[i];
  };

  floatx16 acc[4][kJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < kJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frow = lane % 32, fk = (lane / 32) * 8;
  const int nk = (k + kBK - 1) / kBK;
#pragma unroll
  for (int i = 0; i < kChunks; ++i) load_chunk(0, i);
#pragma unroll
  for (int i = 0; i < kChunks; ++i) store_chunk(0, i);
  if (nk > 1) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) load_chunk(1, i);
  }
  lds_barrier();
  uint4 fa[2][4], fw[2][kJ];
  auto read_fragments = [&](int set, int buf, int ks) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      fa[set][i] = *reinterpret_cast<const uint4*>(&tiles[buf].a[wm * 128 + i * 32 + frow][ks * 16 + fk]);
#pragma unroll
    for (int j = 0; j < kJ; ++j)
      fw[set][j] = *reinterpret_cast<const uint4*>(&tiles[buf].w[wn * kWaveN + j * 32 + frow][ks * 16 + fk]);
  };
  for (int t = 0; t < nk; ++t) {
    const int cur = t & 1;
    const bool st = t + 1 < nk, ld = t + 2 < nk;
    read_fragments(0, cur, 0);
#pragma unroll
    for (int ks = 0; ks < kBK / 16; ++ks) {
      // the next slice's fragments are asked for before this slice's MFMAs, which hide the wait
      if (ks + 1 < kBK / 16) read_fragments((ks + 1) % 2, cur, ks + 1);
      // a part of the next step goes to the other buffer and is asked for again, two steps ahead
#pragma unroll
      for (int c = 0; c < kPerSlice; ++c) {
        if (st) store_chunk(1 - cur, kPerSlice * ks + c);
        if (ld) load_chunk(t + 2, kPerSlice * ks + c);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < kJ; ++j) acc[i][j] = mfma_32x32x16(fa[ks % 2][i], fw[ks % 2][j], acc[i][j]);
    }
    lds_barrier();
  }

  // The tile goes out through LDS, its upper and its lower half in turn, each as two float
  // [128][128 + 4] quarters.  acc[i][j][r] is row wm*128 + i*32 + 8*(r/4) + 4*(lane/32) + r%4 and
  // column wn*kWaveN + j*32 + lane%32 of the tile.
  constexpr int kOutStride = kBN + 4;
  static_assert(2 * sizeof(float) * kBM * kOutStride <= kWideLdsBytes, "two output quarters must fit the operand buffers");
  float* tile_out = reinterpret_cast<float*>(wide_raw);
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    if (half > 0) lds_barrier();
    if (wm == half) {
      const int col0 = wn * kWaveN;
      float* mine = tile_out + (col0 / kBN) * (kBM * kOutStride) + col0 % kBN;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < kJ; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            mine[(i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4) * kOutStride + j * 32 + lane % 32] = acc[i][j][r];
    }
    lds_barrier();
#pragma unroll
    for (int q = 0; q < 2; ++q)
      store_tile<EPI, kThreads>(tile_out + q * (kBM * kOutStride), out, m, n, m0 + 128 * half, n0 + 128 * q, tid);
  }
}

template <int EPI>
int launch_wide(const bf16_t* ap, const bf16_t* wp, void* out, int m, int n, int k, long m_blocks, long n_blocks,
                hipStream_t s) {
  auto kernel = gemm_mfma_wide_kernel<EPI>;
  static bool raised = false;   // per instantiation: allow more than the default dynamic LDS
  if (!raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            static_cast<int>(kWideLdsBytes)) != hipSuccess)
      return fail("gemm_mfma: cannot raise the dynamic LDS limit");
    raised = true;
  }
  kernel<<<dim3(static_cast<unsigned>(m_blocks * n_blocks)), dim3(512), kWideLdsBytes, s>>>(
      ap, wp, out, m, n, k, static_cast<int>(m_blocks), static_cast<int>(n_blocks));
  return 0;
}


template <int EPI>
int launch_tiled(const bf16_t* ap, const bf16_t* wp, void* out, int m, int n, int k, long m_blocks, long n_blocks,
                 hipStream_t s) {
  // Where 256 x 256 tiles fill the CUs round after round (nine tenths of the rounds' places taken),
  // the form with those tiles; with fewer, the idle places of its last round cost more than it gains
  // (measured: 2048 x 28672 x 4096, 3.5 rounds, 633 against 576 us).
  const long wide_blocks = ((m + kWide - 1) / kWide) * ((n + kWide - 1) / kWide);
  const long rounds = (wide_blocks + compute_units() - 1) / compute_units();
  if (wide_blocks * 10 >= rounds * compute_units() * 9)
    return launch_wide<EPI>(ap, wp, out, m, n, k, (m + kWide - 1) / kWide, (n + kWide - 1) / kWide, s);
  // With tiles enough for every CU to have two of them and more, the 256 x 128 tile: a quarter less
  // traffic per FLOP, which is what bounds this kernel.
  const long tall_blocks = (m + 255) / 256;
  if (tall_blocks * n_blocks >= 2L * compute_units()) {
    gemm_mfma_kernel<EPI, 2, 4><<<dim3(static_cast<unsigned>(tall_blocks * n_blocks)), dim3(512), 0, s>>>(
        ap, wp, out, m, n, k, static_cast<int>(tall_blocks), static_cast<int>(n_blocks));
    return 0;
  }
  dim3 grid(static_cast<unsigned>(m_blocks * n_blocks)), block(256);
  // With at most one tile a CU nothing else runs beside a workgroup: then the split form, whose
  // moving and multiplying waves overlap, is the faster one (measured: 29 against 35 us for
  // 2048 x 2048 x 2048); with more tiles two workgroups of the plain form share a CU and do better.
  if (m_blocks * n_blocks <= compute_units()) {
    gemm_mfma_split_kernel<EPI><<<grid, dim3(kSplitThreads), 0, s>>>(ap, wp, out, m, n, k, m_blocks, n_blocks);
    return 0;
  }
  gemm_mfma_kernel<EPI, 2, 2><<<grid, block, 0, s>>>(ap, wp, out, m, n, k, m_blocks, n_blocks);
  return 0;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

extern "C" int bc4g_gemm_mfma(const void* a, const void* w, void* out, int epilogue, int m, int n, int k,
                              void* stream) {
  BC4G_REQUIRE(m >= 0 && n > 0 && k > 0 && k % 8 == 0, "gemm_mfma: K=%d must be a positive multiple of 8 (M=%d N=%d)",
               k, m, n);
  if (m == 0) return 0;
  const long m_blocks = (m + kBM - 1) / kBM, n_blocks = (n + kBN - 1) / kBN;
  BC4G_REQUIRE(m_blocks * n_blocks <= 2147483647L, "gemm_mfma: too many tiles");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bf16_t* ap = static_cast<const bf16_t*>(a);
  const bf16_t* wp = static_cast<const bf16_t*>(w);
  int e = 0;
  switch (epilogue) {
    case kStoreBf16: e = launch_tiled<kStoreBf16>(ap, wp, out, m, n, k, m_blocks, n_blocks, s); break;
    case kStoreF32: e = launch_tiled<kStoreF32>(ap, wp, out, m, n, k, m_blocks, n_blocks, s); break;
    case kAccumF32: e = launch_tiled<kAccumF32>(ap, wp, out, m, n, k, m_blocks, n_blocks, s); break;
    case kSwigluBf16:
      BC4G_REQUIRE(n % 16 == 0, "gemm_mfma: SwiGLU needs blocks of eight gate and eight up rows, N=%d is no multiple of 16", n);
      e = launch_tiled<kSwigluBf16>(ap, wp, out, m, n, k, m_blocks, n_blocks, s);
      break;
    default: return fail("gemm_mfma: unknown epilogue %d", epilogue);
  }
  if (e) return e;
  return check_launch("gemm_mfma");
}
