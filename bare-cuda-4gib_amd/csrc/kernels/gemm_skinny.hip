// out[m, n] = sum_k x[m, k] * w[n, k] for few rows m (a decode step: m <= 64), bfloat16 weights.
//
// The weights are read once, straight from memory into matrix-core registers: a workgroup owns
// 16 output columns n (16 rows of w) and all of k; its 8 waves split k between them, each wave
// feeding 16x16x32 MFMAs with w as the A operand and x as the B operand.  The weights come
// *packed in fragment order*: for every block of 16 rows and every k-step of 32, the 1 KB that a
// wave's 64 lanes load (lane l: row l % 16, k 8 * (l / 16) .. + 7) lies contiguous, blocks and
// k-steps in order -- so every load instruction reads eight whole cache lines and a wave walks
// straight through memory (rows past n and k past the matrix are stored as zeros).  Loads run
// one batch of k-steps ahead of the MFMAs that use them.  The waves' partial sums meet in LDS
// and are added in wave order, so a result does not depend on the number of rows or on timing.
// Where the weight blocks are few and the rows of x more than eight, two workgroups share a block,
// each with half of the rows of x (what a CU can pull through its cache bounds the kernel, so the
// pulling is spread).
//
// What comes in (XMODE):
//   plain    x is bfloat16 [m, k].  The B operand's own pattern (a lane group reads 16 bytes of
//            each of 16 rows) keeps the texture path busy four times as long as a load of whole
//            cache lines, and with 64 rows x is four times the weights' traffic: so x comes in row
//            by row (eight or sixteen lanes read a row's part of the batch) and is turned into
//            operand order through a buffer in LDS that belongs to the wave -- no barrier, and the
//            next batch's loads are in flight meanwhile.
//   normed   x is the float residual stream (rows taken through `rows` if given) and RMSNorm is
//            fused (up to 16 rows): while the first weights are already on their way, the
//            workgroup writes bf16(x * g) into LDS and sums x^2 per row; the MFMAs read their B
//            operand from LDS, and the row's rsqrt(mean(x^2) + eps) -- a factor common to the
//            whole row -- multiplies the finished sum.
//   prenormed  x is bfloat16(residual * g), written by the product that last added to the residual
//            (below), together with parts of every row's sum of squares: the row's scale is worked out
//            from the parts while the weights are on their way and multiplies the finished sum -- the
//            norm costs neither a kernel of its own nor the staging of the float rows.
// What goes out (EPI): bfloat16 or float stored; float added into the residual stream; SwiGLU,
// when every 16 rows of w are eight gate rows followed by the eight up rows of the same outputs; or
// rotary positions and the cache write, when w holds query, key and value heads with every head's
// rows reordered in blocks of 16 (eight dimensions, then their rotation partners): queries are
// stored rotated, keys rotated into their page, values into theirs.  The epilogue that adds into the
// residual stream can prepare the RMSNorm that follows (emit): it also stores bfloat16(new residual * g)
// and, per row, the sum of squares over its 16 columns -- parts that the next product adds up in
// block order, so the result does not depend on timing.
#include <type_traits>
#include <math.h>

#include "api.h"
#include "mfma.h"

namespace bc4g {
namespace {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kRedPad = 17;
constexpr int kStagePad = 8;     // bf16 elements appended to each staged row of x

enum Epilogue : int { kStoreBf16 = 0, kStoreF32 = 1, kAccumF32 = 2, kSwigluBf16 = 3, kRopeKvBf16 = 4 };

struct RopeKvArgs {
  const int32_t* positions;   // [m]
  const int32_t* slot_map;    // [m] page * page_tokens + offset
  bf16_t* k_cache;            // [pages, n_kv, page_tokens, d], or every [page_tokens, d] in fragment order
  bf16_t* v_cache;            // [pages, n_kv, d, page_tokens], or likewise
  int n_heads, n_kv_heads, head_dim, rotary_dim, page_tokens, write_kv;
  int fragment_order;         // how the cache's pages are laid out (cache_fragment_order)
  float theta;
};
enum XMode : int { kPlain = 0, kNormedG16 = 1, kNormedG32 = 2 };   // norm scale g in bfloat16 / float

struct SkinnyArgs {
  const void* x;            // bf16 [m, k], or float [*, k] in the normed modes
  const int32_t* rows;      // normed modes: row m of the product reads x[rows[m]] (null: x[m])
  const void* g;            // normed modes: RMSNorm scale [k]
  const bf16_t* w;          // packed: [ceil(n / 16)][ceil(k / 32)][64 lanes][8]
  void* out;
  int m, n, k, n_out;
  int rows_per_block;       // plain mode: blockIdx.y takes rows y * rows_per_block .. of x and out (0: all rows)
  int m_stage;              // normed modes: rows of x staged in LDS (m rounded up to 4)
  float eps;
  // prenormed x (plain mode): parts [ssq_blocks][ssq_stride] of the rows' sums of squares (null: x as it is)
  const float* ssq_parts;
  int ssq_blocks, ssq_stride;
  // kAccumF32: what the RMSNorm after this product needs (emit_g null: nothing)
  const void* emit_g;       // [n] its scale, bfloat16 or float (emit_g_f32)
  bf16_t* emit_x;           // [m, n] bfloat16(new residual * g)
  float* emit_ssq;          // [ceil(n / 16)][emit_stride]: block b's part of row r's sum of squares
  int emit_g_f32, emit_stride;
  RopeKvArgs rope;          // kRopeKvBf16 only
};

__device__ inline uint32_t pack2(float a, float b) {
  return static_cast<uint32_t>(bf16_bits_from_float(a)) | (static_cast<uint32_t>(bf16_bits_from_float(b)) << 16);
}

template <int MT, int EPI, int XMODE, int U>
// (The normed form keeps to 80 registers, so that three workgroups share a CU and all the blocks of
// a 5,632 x 2 wide gate-up matrix are in flight at once.)
__global__ __launch_bounds__(kThreads, (XMODE != kPlain || (MT == 1 && U == 2)) ? 6 : 4) void gemm_skinny_kernel(const SkinnyArgs args) {
  constexpr bool kNormed = XMODE != kPlain;
  // Where the weight blocks are too few to occupy the CUs, the rows are shared out over blockIdx.y:
  // such a workgroup sees its own rows only, as if they were the whole batch.
  SkinnyArgs a = args;
  if (!kNormed && args.rows_per_block > 0) {
    const long row0 = static_cast<long>(blockIdx.y) * args.rows_per_block;
    a.m = min(args.rows_per_block, args.m - static_cast<int>(row0));
    a.x = static_cast<const bf16_t*>(args.x) + row0 * args.k;
    if constexpr (EPI == kStoreBf16) a.out = static_cast<bf16_t*>(args.out) + row0 * args.n;
    else if constexpr (EPI == kSwigluBf16) a.out = static_cast<bf16_t*>(args.out) + row0 * (args.n / 2);
    else if constexpr (EPI == kRopeKvBf16) {
      a.out = static_cast<bf16_t*>(args.out) + row0 * args.rope.n_heads * args.rope.head_dim;
      a.rope.positions = args.rope.positions ? args.rope.positions + row0 : nullptr;
      a.rope.slot_map = args.rope.slot_map ? args.rope.slot_map + row0 : nullptr;
    } else a.out = static_cast<float*>(args.out) + row0 * args.n;
    if (args.ssq_parts) a.ssq_parts = args.ssq_parts + row0;
    if (EPI == kAccumF32 && args.emit_g) {
      a.emit_x = args.emit_x + row0 * args.n;
      a.emit_ssq = args.emit_ssq + row0;
    }
  }
  constexpr bool kTurned = !kNormed;                      // x reaches operand order through LDS
  constexpr int kPieces = 4 * U;                       // 16-byte pieces of a row in one batch of k-steps
  static_assert(!kNormed || MT == 1, "the fused norm handles one tile of rows");
  static_assert(!kTurned || 64 % kPieces == 0, "a load instruction covers whole rows of a batch");
  static_assert(!kTurned || kPieces >= 8, "the buffer's swizzle (piece ^ row % 8) must stay inside a row's pieces");
  // The waves' partial sums, and before them (kTurned) every wave's buffer for x: the same memory.
  typedef float Red[MT][16][kRedPad];
  constexpr int kRedBytes = kWaves * static_cast<int>(sizeof(Red));
  constexpr int kTurnBytes = kTurned ? kWaves * MT * 16 * kPieces * 16 : 0;
  __shared__ __align__(16) unsigned char pool[kRedBytes > kTurnBytes ? kRedBytes : kTurnBytes];
  Red* red = reinterpret_cast<Red*>(pool);
  __shared__ float ssq_row[16];
  extern __shared__ __align__(16) unsigned char stage_raw[];   // normed: bf16 [m_stage][k + kStagePad]
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: k ranges and bases stay scalar
  const int col = lane % 16, grp = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int k = a.k, m = a.m;

  // every wave's part of k starts on a cache line of x (64 elements), whatever the number of rows:
  // the order of the additions, and so the rounding, is the same in every form of the kernel
  const int chunk = ((k + kWaves * 64 - 1) / (kWaves * 64)) * 64;
  const int k_begin = wave * chunk;
  const int k_end = min(k, k_begin + chunk);

  floatx4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // this workgroup's block of 16 rows in the packed weights: k-step ks at wblock + ks * 512 elements
  // (a scalar base and a 32-bit lane offset, so the loads of a batch differ in their scalar part only)
  const int ksteps_total = (k + 31) / 32;
  const bf16_t* wblock = a.w + static_cast<long>(blockIdx.x) * ksteps_total * (kWave * 8);
  const int wlane = lane * 8;

  // where this lane's B operand comes from
  const bf16_t* xptr[MT];
  bool xrow_ok[MT];
  const int stage_stride = k + kStagePad;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int row = t * 16 + col;
    xrow_ok[t] = row < m;
    if constexpr (kNormed) {
      xptr[t] = reinterpret_cast<const bf16_t*>(stage_raw) + static_cast<long>(min(row, a.m_stage - 1)) * stage_stride;
    } else {
      xptr[t] = static_cast<const bf16_t*>(a.x) + static_cast<long>(row) * k;
    }
  }

  // The float sums that the product is added to (the residual stream) are asked for now, not
  // after the weights: item j of a thread is output (threadIdx.x + j * kThreads) of the block.
  constexpr int kAccItems = (MT * 256 + kThreads - 1) / kThreads;
  float prev[kAccItems];
  if constexpr (EPI == kAccumF32) {
#pragma unroll
    for (int j = 0; j < kAccItems; ++j) {
      const int idx = threadIdx.x + j * kThreads;
      const int row = idx / 16, gn = n0 + idx % 16;
      prev[j] = (idx < MT * 256 && row < m && gn < a.n) ? static_cast<const float*>(a.out)[static_cast<long>(row) * a.n + gn] : 0.f;
    }
  }

  // The rotation a thread will apply in the epilogue (its output's angle: position and pair are
  // known now) and the place in the cache it will write to are worked out while the weights are
  // on their way: item j of a thread is pair (threadIdx.x + j * kThreads) % 8 of row ... / 8.
  constexpr int kRopeItems = (MT * 128 + kThreads - 1) / kThreads;
  float rope_cs[kRopeItems], rope_sn[kRopeItems];
  int rope_slot[kRopeItems];
  if constexpr (EPI == kRopeKvBf16) {
    const RopeKvArgs& r = a.rope;
    const int head = n0 / r.head_dim;
    const bool is_v = head >= r.n_heads + r.n_kv_heads;
#pragma unroll
    for (int j = 0; j < kRopeItems; ++j) {
      const int idx = threadIdx.x + j * kThreads;
      const int row = idx / 8, nl = idx % 8;
      const bool live = idx < MT * 128 && row < m;
      rope_cs[j] = 1.f;
      rope_sn[j] = 0.f;
      if (live && r.rotary_dim > 0 && !is_v) {
        const int pair = (n0 % r.head_dim) / 2 + nl;            // 8 * block + nl
        const float inv_freq = 1.0f / powf(r.theta, (2.0f * static_cast<float>(pair)) / static_cast<float>(r.head_dim));
        sincosf(static_cast<float>(r.positions[row]) * inv_freq, &rope_sn[j], &rope_cs[j]);
      }
      rope_slot[j] = (live && head >= r.n_heads && r.write_kv) ? r.slot_map[row] : 0;
    }
  }

  // prenormed x: every row's sum of squares from its parts.  Eight threads a row, thread j adding
  // the parts of blocks j, j + 8, ... in ascending order; the eight sums meet in LDS and are added in
  // order of j after the product: the order of the additions, and so the rounding, is the same for
  // every number of rows.  (After the first weights have been asked for.)  How many parts a thread asks
  // for together, by what was measured inside a model: sixteen -- one way to memory and back for 128
  // parts instead of four -- up to 8 rows in the kernels that serve those (four k-steps a turn, and the
  // SwiGLU product: a decode step at TinyLlama's sizes 1.000 -> 0.983 ms at 8 rows, 0.922 -> 0.917 at
  // one), four otherwise (with sixteen or eight a step of 16 rows was 0.4-0.8 % longer, and the other
  // kernels of two k-steps a turn spilled).
  constexpr int kPartSums = 8;
  __shared__ float part_sum[kPartSums][MT * 16];
  const bool prenormed = !kNormed && a.ssq_parts != nullptr;
  auto sum_parts = [&]() {
    if (prenormed && threadIdx.x < kPartSums * MT * 16) {
      const int row = threadIdx.x % (MT * 16), j0 = threadIdx.x / (MT * 16);
      float ss = 0.f;
      if (row < m) {
        const float* p = a.ssq_parts + row;
        auto chain = [&](auto ahead) {
          constexpr int kAhead = decltype(ahead)::value;
          for (int b0 = j0; b0 < a.ssq_blocks; b0 += kAhead * kPartSums) {
            float part[kAhead];
#pragma unroll
            for (int i = 0; i < kAhead; ++i) {
              const int b = b0 + i * kPartSums;
              part[i] = b < a.ssq_blocks ? p[static_cast<long>(b) * a.ssq_stride] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < kAhead; ++i) ss += part[i];      // (in ascending order; a part that is not there adds 0)
          }
        };
        if ((U == 4 || EPI == kSwigluBf16) && m <= 8) chain(std::integral_constant<int, 16>{});
        else chain(std::integral_constant<int, 4>{});
      }
      part_sum[j0][row] = ss;
    }
  };

  // kTurned: load i of a batch brings piece (i * 64 + lane) % kPieces of row (i * 64 + lane) / kPieces;
  // in the wave's buffer piece p of row r lies at r * kPieces + (p ^ (r % 8)), which keeps both the
  // row-wise writes and the operand-wise reads (16 rows at one piece) off each other's banks.
  constexpr int kRowsPerLoad = kTurned ? 64 / kPieces : 1;
  const int turn_row = lane / kPieces, turn_piece = lane % kPieces;
  const bf16_t* turn_src = static_cast<const bf16_t*>(a.x) + static_cast<long>(turn_row) * k + turn_piece * 8;
  uint4* turn = reinterpret_cast<uint4*>(pool) + wave * (MT * 16 * kPieces);

  struct Batch {
    uint4 w[U];
    uint4 x[kNormed ? 1 : MT][kNormed ? 1 : U];
  };
  // A batch that lies whole inside the wave's part of k can be loaded without a condition anywhere (rows past m read
  // the last row: their results are never stored).  The compiler counts outstanding loads by instruction: where a load
  // may be skipped it cannot know how many were issued after the ones it waits for and waits for all of them, and a
  // copy from one set of registers to the other waits for the load it copies -- every batch then waits for the batch
  // asked for just before it.  With 32 rows a workgroup, whole batches are loaded so and multiplied from the
  // registers they were loaded into, two a turn (64 rows as two workgroups of 32: the down projection of 5,632
  // 10.9 -> 9.0 us, the others 2-4 % less); with 16 rows the plain loop is the faster one (4.2 against 4.7 us for a
  // 2,048 x 2,048 block of weights), and with 48 and 64 rows a workgroup the second set of registers does not fit the
  // 128 a wave has (spilled, the q|k|v product of 64 rows and 4,096 columns took 127 instead of 44 us).
  constexpr bool kPingPong = MT == 2;
  const int last_row_offset = (m - 1) * k;              // (m <= 64 rows: an int)
  int turn_offset[kTurned ? MT * U : 1];
  if constexpr (kTurned) {
#pragma unroll
    for (int i = 0; i < MT * U; ++i) turn_offset[i] = min((turn_row + i * kRowsPerLoad) * k, last_row_offset) + turn_piece * 8;
  }
  const bf16_t* xptr_any[MT];                           // (the row itself, or the last row for rows past m)
#pragma unroll
  for (int t = 0; t < MT; ++t) xptr_any[t] = (kNormed || xrow_ok[t]) ? xptr[t] : static_cast<const bf16_t*>(a.x) + last_row_offset;
  auto load_whole = [&](Batch& b, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      b.w[u] = load16(wblock + static_cast<long>(k0 / 32 + u) * (kWave * 8) + wlane);
      if constexpr (!kNormed && !kTurned) {
#pragma unroll
        for (int t = 0; t < MT; ++t) b.x[t][u] = load16(xptr_any[t] + k0 + 32 * u + 8 * grp);
      }
    }
    if constexpr (kTurned) {
#pragma unroll
      for (int i = 0; i < MT * U; ++i) b.x[i / U][i % U] = load16(static_cast<const bf16_t*>(a.x) + turn_offset[i] + k0);
    }
  };
  auto load = [&](Batch& b, int k0) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = k0 + 32 * u + 8 * grp;
      const bool ok = kk < k_end;
      b.w[u] = k0 + 32 * u < k_end ? load16(wblock + static_cast<long>(k0 / 32 + u) * (kWave * 8) + wlane) : zero16();
      if constexpr (!kNormed && !kTurned) {
#pragma unroll
        for (int t = 0; t < MT; ++t) b.x[t][u] = (ok && xrow_ok[t]) ? load16(xptr[t] + kk) : zero16();
      }
    }
    if constexpr (kTurned) {
      const bool k_ok = k0 + turn_piece * 8 < k_end;
#pragma unroll
      for (int i = 0; i < MT * U; ++i) {
        const bool ok = k_ok && turn_row + i * kRowsPerLoad < m;
        b.x[i / U][i % U] = ok ? load16(turn_src + static_cast<long>(i * kRowsPerLoad) * k + k0) : zero16();
      }
    }
  };
  auto compute = [&](const Batch& b, int k0) {
    if constexpr (kTurned) {
#pragma unroll
      for (int i = 0; i < MT * U; ++i) {
        const int row = turn_row + i * kRowsPerLoad;
        turn[row * kPieces + (turn_piece ^ (row % 8))] = b.x[i / U][i % U];
      }
      // the wave's own lanes wrote what its lanes now read: LDS serves a wave's accesses in order
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        uint4 xb;
        if constexpr (kNormed) {
          const int kk = k0 + 32 * u + 8 * grp;
          xb = kk < k_end ? *reinterpret_cast<const uint4*>(xptr[t] + kk) : zero16();
        } else if constexpr (kTurned) {
          xb = turn[(t * 16 + col) * kPieces + ((4 * u + grp) ^ (col % 8))];
        } else {
          xb = b.x[t][u];
        }
        acc[t] = mfma_16x16x32(b.w[u], xb, acc[t]);
      }
    }
    if constexpr (kTurned) {                             // read before the next batch is written
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  };

  constexpr int kStep = 32 * U;
  Batch cur, nxt;

  if constexpr (kNormed) {
    // Stage bf16(x * g): wave w takes rows w, w + 8; a lane takes 8 elements of each 512.  The
    // loads of x and g are issued first and the first weights right after them: loads come back
    // in the order they were issued, so the (cached) x arrives while the weights are on their way.
    constexpr int kStageIters = 2;                       // 1024 elements of a row per round
    bf16_t* stage = reinterpret_cast<bf16_t*>(stage_raw);
    bool first = true;
    for (int row = wave; row < a.m_stage; row += kWaves) {
      float ss = 0.f;
      const bool live = row < m;
      const long src = (live && a.rows) ? a.rows[row] : row;
      const float* xr = static_cast<const float*>(a.x) + src * k;
      for (int kb = 0; kb < k; kb += 512 * kStageIters) {
        uint4 x0[kStageIters], x1[kStageIters], g0[kStageIters], g1[kStageIters];
#pragma unroll
        for (int it = 0; it < kStageIters; ++it) {
          const int kk = kb + it * 512 + lane * 8;
          const bool ok = live && kk < k;
          x0[it] = ok ? load16(xr + kk) : zero16();
          x1[it] = ok ? load16(xr + kk + 4) : zero16();
          if constexpr (XMODE == kNormedG16) {
            g0[it] = ok ? load16(static_cast<const bf16_t*>(a.g) + kk) : zero16();
          } else {
            g0[it] = ok ? load16(static_cast<const float*>(a.g) + kk) : zero16();
            g1[it] = ok ? load16(static_cast<const float*>(a.g) + kk + 4) : zero16();
          }
        }
        if (first) {                                       // the first weights follow the first x
          if (k_begin < k_end) load(cur, k_begin);
          first = false;
        }
#pragma unroll
        for (int it = 0; it < kStageIters; ++it) {
          const int kk = kb + it * 512 + lane * 8;
          if (kk >= k) continue;
          const float xv[8] = {__uint_as_float(x0[it].x), __uint_as_float(x0[it].y), __uint_as_float(x0[it].z),
                               __uint_as_float(x0[it].w), __uint_as_float(x1[it].x), __uint_as_float(x1[it].y),
                               __uint_as_float(x1[it].z), __uint_as_float(x1[it].w)};
          float gv[8];
          if constexpr (XMODE == kNormedG16) {
            const uint32_t gr[4] = {g0[it].x, g0[it].y, g0[it].z, g0[it].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              gv[2 * i] = __uint_as_float(gr[i] << 16);
              gv[2 * i + 1] = __uint_as_float(gr[i] & 0xffff0000u);
            }
          } else {
            const uint32_t gr[8] = {g0[it].x, g0[it].y, g0[it].z, g0[it].w, g1[it].x, g1[it].y, g1[it].z, g1[it].w};
#pragma unroll
            for (int i = 0; i < 8; ++i) gv[i] = __uint_as_float(gr[i]);
          }
#pragma unroll
          for (int i = 0; i < 8; ++i) ss += xv[i] * xv[i];
          *reinterpret_cast<uint4*>(stage + static_cast<long>(row) * stage_stride + kk) =
              make_uint4(pack2(xv[0] * gv[0], xv[1] * gv[1]), pack2(xv[2] * gv[2], xv[3] * gv[3]),
                         pack2(xv[4] * gv[4], xv[5] * gv[5]), pack2(xv[6] * gv[6], xv[7] * gv[7]));
        }
      }
      ss = wave_sum(ss);
      if (lane == 0 && row < 16) ssq_row[row] = ss;
    }
    if (first && k_begin < k_end) load(cur, k_begin);      // a wave without a row to stage
    lds_barrier();                                         // (the weights stay in flight)
  } else {
    if (k_begin < k_end) load(cur, k_begin);
    sum_parts();
  }

  int k0 = k_begin;
  while (kPingPong && k0 + 3 * kStep <= k_end) {
    load_whole(nxt, k0 + kStep);
    compute(cur, k0);
    load_whole(cur, k0 + 2 * kStep);
    compute(nxt, k0 + kStep);
    k0 += 2 * kStep;
  }
  for (; k0 < k_end; k0 += kStep) {
    const int next = k0 + kStep;
    if (kPingPong && next + kStep <= k_end) load_whole(nxt, next);
    else if (next < k_end) load(nxt, next);
    compute(cur, k0);
    if (next < k_end) cur = nxt;
  }

  if constexpr (kTurned) __syncthreads();               // the partial sums take the buffers' place
  // acc[t][r] is the partial sum for output column n0 + 4*grp + r and row t*16 + col
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][4 * grp + r][col] = acc[t][r];
  __syncthreads();

  constexpr bool kPaired = EPI == kSwigluBf16 || EPI == kRopeKvBf16;   // columns nl and nl + 8 belong together
  constexpr int kCols = kPaired ? 8 : 16;
  constexpr int kItems = (MT * 16 * kCols + kThreads - 1) / kThreads;
#pragma unroll
  for (int j = 0; j < kItems; ++j) {
    const int idx = threadIdx.x + j * kThreads;
    const int nl = idx % kCols, row = idx / kCols;
    const int gn = n0 + nl;
    const bool live = idx < MT * 16 * kCols && row < m && gn < a.n;
    // (the adding epilogue goes on with every lane: its lanes may have sums of squares to exchange)
    if (EPI != kAccumF32 && !live) continue;
    float sum = 0.f, partner = 0.f;
    if (live) {
#pragma unroll
      for (int wv = 0; wv < kWaves; ++wv) sum += red[wv][row / 16][nl][row % 16];
      if constexpr (kPaired) {
#pragma unroll
        for (int wv = 0; wv < kWaves; ++wv) partner += red[wv][row / 16][nl + 8][row % 16];
      }
    }
    if (kNormed || prenormed) {
      float ssq = 0.f;
      if (live) {
        if (prenormed) {
#pragma unroll
          for (int j2 = 0; j2 < kPartSums; ++j2) ssq += part_sum[j2][row];
        } else {
          ssq = ssq_row[row];
        }
      }
      const float scale = live ? 1.0f / sqrtf(ssq / static_cast<float>(k) + a.eps) : 0.f;
      sum *= scale;
      partner *= scale;
    }
    if constexpr (EPI == kStoreBf16) {
      static_cast<bf16_t*>(a.out)[static_cast<long>(row) * a.n + gn] = from_float<bf16_t>(sum);
    } else if constexpr (EPI == kStoreF32) {
      static_cast<float*>(a.out)[static_cast<long>(row) * a.n + gn] = sum;
    } else if constexpr (EPI == kAccumF32) {
      const float nv = prev[j] + sum;
      if (live) static_cast<float*>(a.out)[static_cast<long>(row) * a.n + gn] = nv;
      if (a.emit_g != nullptr) {
        // for the RMSNorm that follows: bf16(new residual * g), and this block's part of the row's sum
        // of squares (a row's 16 columns lie in 16 neighbouring lanes)
        float sq = 0.f;
        if (live) {
          const float g = a.emit_g_f32 ? static_cast<const float*>(a.emit_g)[gn]
                                       : to_float(static_cast<const bf16_t*>(a.emit_g)[gn]);
          a.emit_x[static_cast<long>(row) * a.n + gn] = from_float<bf16_t>(nv * g);
          sq = nv * nv;
        }
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) sq += __shfl_xor(sq, off, kWave);
        if (nl == 0 && idx < MT * 256 && row < m) a.emit_ssq[static_cast<long>(blockIdx.x) * a.emit_stride + row] = sq;
      }
    } else if constexpr (EPI == kSwigluBf16) {
      // block b = n0 / 16 holds gates and ups of outputs 8b .. 8b + 7
      const long o = static_cast<long>(row) * (a.n / 2) + (n0 / 2 + nl);
      static_cast<bf16_t*>(a.out)[o] = from_float<bf16_t>(silu_quick(sum) * partner);
    } else {
      const RopeKvArgs& r = a.rope;
      const int d = r.head_dim;
      const int head = n0 / d, in_head = n0 % d + nl;         // the pair lies at in_head and in_head + 8
      float lo = sum, hi = partner;
      const bool is_v = head >= r.n_heads + r.n_kv_heads;
      if (r.rotary_dim > 0 && !is_v) {
        const float cs = rope_cs[j], sn = rope_sn[j], l0 = lo, h0 = hi;
        lo = l0 * cs - h0 * sn;
        hi = h0 * cs + l0 * sn;
      }
      if (head < r.n_heads) {
        bf16_t* q = static_cast<bf16_t*>(a.out) + (static_cast<long>(row) * r.n_heads + head) * d + in_head;
        q[0] = from_float<bf16_t>(lo);
        q[8] = from_float<bf16_t>(hi);
      } else if (r.write_kv) {
        const int kvh = is_v ? head - r.n_heads - r.n_kv_heads : head - r.n_heads;
        const int slot = rope_slot[j];
        const long page = slot / r.page_tokens, off = slot % r.page_tokens;
        const long region = (page * r.n_kv_heads + kvh) * d * r.page_tokens;
        if (r.fragment_order) {
          bf16_t* dst = (is_v ? r.v_cache : r.k_cache) + region;
          const int o = static_cast<int>(off);
          dst[is_v ? frag_v_offset(o, in_head, d) : frag_k_offset(o, in_head, d)] = from_float<bf16_t>(lo);
          dst[is_v ? frag_v_offset(o, in_head + 8, d) : frag_k_offset(o, in_head + 8, d)] = from_float<bf16_t>(hi);
        } else if (is_v) {
          bf16_t* dst = r.v_cache + region + in_head * r.page_tokens + off;
          dst[0] = from_float<bf16_t>(lo);
          dst[8L * r.page_tokens] = from_float<bf16_t>(hi);
        } else {
          bf16_t* dst = r.k_cache + region + off * d + in_head;
          dst[0] = from_float<bf16_t>(lo);
          dst[8] = from_float<bf16_t>(hi);
        }
      }
    }
  }
}

constexpr int kMaxStageBytes = 96 * 1024;
constexpr int kSplitMinRows = 8;

template <int EPI, int XMODE>
int launch(const SkinnyArgs& a, hipStream_t s) {
  const int mt = (a.m + 15) / 16;
  dim3 grid((a.n + 15) / 16), block(kThreads);
  if constexpr (XMODE != kPlain) {
    if (mt != 1) return fail("gemm_skinny: the fused norm takes at most 16 rows, got %d", a.m);
    const size_t stage = static_cast<size_t>(a.m_stage) * (a.k + kStagePad) * 2;
    if (stage > kMaxStageBytes) return fail("gemm_skinny: %d rows of k=%d do not fit the staging buffer", a.m, a.k);
    auto kernel = gemm_skinny_kernel<1, EPI, XMODE, 4>;
    static bool raised = false;   // per instantiation: allow more than the default dynamic LDS
    if (!raised) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              kMaxStageBytes) != hipSuccess)
        return fail("gemm_skinny: cannot raise the dynamic LDS limit");
      raised = true;
    }
    kernel<<<grid, block, stage, s>>>(a);
  } else {
    // Every workgroup reads all its rows of x, and what a CU can pull through its cache is what bounds
    // the kernel once x is as large as the block's weights (16 rows).  Where the weight blocks are
    // few (up to one a CU: n = 4,096), two workgroups share a block's rows: each pulls half of
    // x, and the block's weights are read twice, once of it from L2 (measured at TinyLlama's sizes:
    // 1.80 -> 1.51 ms a step at 64 rows, 1.36 -> 1.26 at 32, 1.15 -> 1.12 at 16; four workgroups a
    // block, or splitting the wide gate-up product too, are no faster).
    SkinnyArgs b = a;
    int tiles = mt;
    if (a.m > kSplitMinRows && static_cast<int>(grid.x) <= compute_units()) {
      b.rows_per_block = (a.m + 1) / 2;
      tiles = (b.rows_per_block + 15) / 16;
      grid.y = 2;
    }
    switch (tiles) {
      // k-steps per batch chosen so that two batches of operands fit 128 registers (two workgroups a CU)
      case 1:
        // (a wide product's many workgroups, more than two a CU: with fewer k-steps in flight each they
        // need half the registers, and all of them are on the CUs at once -- the gate-up product of 8
        // rows after a prepared norm: a decode step 1.020 -> 0.990 ms)
        if (static_cast<int>(grid.x) > 2 * compute_units()) gemm_skinny_kernel<1, EPI, XMODE, 2><<<grid, block, 0, s>>>(b);
        else gemm_skinny_kernel<1, EPI, XMODE, 4><<<grid, block, 0, s>>>(b);
        break;
      case 2: gemm_skinny_kernel<2, EPI, XMODE, 2><<<grid, block, 0, s>>>(b); break;
      case 3: gemm_skinny_kernel<3, EPI, XMODE, 2><<<grid, block, 0, s>>>(b); break;
      case 4: gemm_skinny_kernel<4, EPI, XMODE, 2><<<grid, block, 0, s>>>(b); break;
      default: return fail("gemm_skinny: M=%d is beyond 64 rows", a.m);
    }
  }
  return check_launch("gemm_skinny");
}

template <int XMODE>
int launch_epilogue(SkinnyArgs& a, int epilogue, hipStream_t s) {
  a.n_out = a.n;
  switch (epilogue) {
    case kStoreBf16: return launch<kStoreBf16, XMODE>(a, s);
    case kStoreF32: return launch<kStoreF32, XMODE>(a, s);
    case kAccumF32:
      if constexpr (XMODE == kPlain) return launch<kAccumF32, XMODE>(a, s);
      else return fail("gemm_skinny: adding into the stream that is being normed is not supported");
    case kSwigluBf16: return launch<kSwigluBf16, XMODE>(a, s);
    case kRopeKvBf16: return launch<kRopeKvBf16, XMODE>(a, s);
    default: return fail("gemm_skinny: unknown epilogue %d", epilogue);
  }
}

int check_common(const char* what, int m, int max_m, int n, int k, int epilogue) {
  BC4G_REQUIRE(m >= 0 && m <= max_m, "%s: M=%d must be at most %d", what, m, max_m);
  BC4G_REQUIRE(n > 0 && k > 0 && k % 8 == 0, "%s: K=%d must be a positive multiple of 8 (N=%d)", what, k, n);
  BC4G_REQUIRE(epilogue != kSwigluBf16 || n % 16 == 0,
               "%s: SwiGLU needs blocks of eight gate and eight up rows, N=%d is no multiple of 16", what, n);
  return 0;
}

int check_rope(const char* what, const RopeKvArgs& r, int n) {
  BC4G_REQUIRE(r.n_heads > 0 && r.n_kv_heads > 0 && r.head_dim > 0 && r.head_dim % 16 == 0,
               "%s: bad head sizes %d/%d x %d (head_dim must be a multiple of 16)", what, r.n_heads, r.n_kv_heads,
               r.head_dim);
  BC4G_REQUIRE(n == (r.n_heads + 2 * r.n_kv_heads) * r.head_dim, "%s: N=%d is not (heads + 2 kv heads) * head_dim", what, n);
  BC4G_REQUIRE(r.rotary_dim == 0 || (r.rotary_dim == r.head_dim && r.positions && r.theta > 0.f),
               "%s: the rotation must cover the whole head (rotary_dim %d, head_dim %d)", what, r.rotary_dim, r.head_dim);
  BC4G_REQUIRE(!r.write_kv || (r.slot_map && r.k_cache && r.v_cache && r.page_tokens > 0),
               "%s: cache write asked for without a cache", what);
  return 0;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

namespace bc4g {
namespace {
SkinnyArgs plain_args(const void* x, const void* w, void* out, int m, int n, int k) {
  SkinnyArgs a{};
  a.x = x;
  a.w = static_cast<const bf16_t*>(w);
  a.out = out;
  a.m = m;
  a.n = n;
  a.k = k;
  a.n_out = n;
  return a;
}

int check_parts(const char* what, const float* ssq_parts, int ssq_blocks, int ssq_stride, int m, float eps) {
  BC4G_REQUIRE(ssq_parts != nullptr && ssq_blocks > 0 && ssq_stride >= m, "%s: the sums of squares need %d parts of at least %d rows",
               what, ssq_blocks, m);
  BC4G_REQUIRE(eps >= 0.f, "%s: eps must not be negative", what);
  return 0;
}
}  // namespace
}  // namespace bc4g

extern "C" int bc4g_gemm_skinny(const void* x, const void* w, void* out, int epilogue, int m, int n, int k,
                                void* stream) {
  if (int e = check_common("gemm_skinny", m, 64, n, k, epilogue)) return e;
  BC4G_REQUIRE(epilogue != kRopeKvBf16, "gemm_skinny: use bc4g_gemm_skinny_qkv for the rotary epilogue");
  if (m == 0) return 0;
  SkinnyArgs a = plain_args(x, w, out, m, n, k);
  return launch_epilogue<kPlain>(a, epilogue, static_cast<hipStream_t>(stream));
}

// out (the float residual stream, [m, n]) += x w^T, and what the RMSNorm after it needs: emit_x
// [m, n] = bfloat16(new residual * g) and emit_ssq [ceil(n / 16)][emit_stride], block b's part of
// every row's sum of squares.
extern "C" int bc4g_gemm_skinny_emit(const void* x, const void* w, float* out, const void* g, int g_dtype, void* emit_x,
                                     float* emit_ssq, int emit_stride, int m, int n, int k, void* stream) {
  if (int e = check_common("gemm_skinny_emit", m, 64, n, k, kAccumF32)) return e;
  BC4G_REQUIRE(g && emit_x && emit_ssq && emit_stride >= m, "gemm_skinny_emit: the norm's scale and both outputs are needed");
  BC4G_REQUIRE(g_dtype == kBF16 || g_dtype == kF32, "gemm_skinny_emit: unknown norm scale dtype %d", g_dtype);
  if (m == 0) return 0;
  SkinnyArgs a = plain_args(x, w, out, m, n, k);
  a.emit_g = g;
  a.emit_g_f32 = g_dtype == kF32 ? 1 : 0;
  a.emit_x = static_cast<bf16_t*>(emit_x);
  a.emit_ssq = emit_ssq;
  a.emit_stride = emit_stride;
  return launch<kAccumF32, kPlain>(a, static_cast<hipStream_t>(stream));
}

// x is bfloat16(residual * g) and ssq_parts the parts of the rows' sums of squares, as
// bc4g_gemm_skinny_emit leaves them: out = rmsnorm(residual) w^T with the epilogues of bc4g_gemm_skinny
// except the adding one.
extern "C" int bc4g_gemm_skinny_prenormed(const void* x, const float* ssq_parts, int ssq_blocks, int ssq_stride, float eps,
                                          const void* w, void* out, int epilogue, int m, int n, int k, void* stream) {
  if (int e = check_common("gemm_skinny_prenormed", m, 64, n, k, epilogue)) return e;
  if (int e = check_parts("gemm_skinny_prenormed", ssq_parts, ssq_blocks, ssq_stride, m, eps)) return e;
  BC4G_REQUIRE(epilogue != kAccumF32 && epilogue != kRopeKvBf16, "gemm_skinny_prenormed: epilogue %d is not supported here",
               epilogue);
  if (m == 0) return 0;
  SkinnyArgs a = plain_args(x, w, out, m, n, k);
  a.ssq_parts = ssq_parts;
  a.ssq_blocks = ssq_blocks;
  a.ssq_stride = ssq_stride;
  a.eps = eps;
  return launch_epilogue<kPlain>(a, epilogue, static_cast<hipStream_t>(stream));
}

extern "C" int bc4g_gemm_skinny_normed(const float* x, const int32_t* rows, const void* g, int g_dtype,
                                       float eps, const void* w, void* out, int epilogue, int m, int n, int k,
                                       void* stream) {
  if (int e = check_common("gemm_skinny_normed", m, 16, n, k, epilogue)) return e;
  BC4G_REQUIRE(epilogue != kAccumF32 && epilogue != kRopeKvBf16, "gemm_skinny_normed: epilogue %d is not supported here",
               epilogue);
  if (m == 0) return 0;
  SkinnyArgs a = plain_args(x, w, out, m, n, k);
  a.rows = rows;
  a.g = g;
  a.m_stage = ((m + 3) / 4) * 4;
  a.eps = eps;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (g_dtype == kBF16) return launch_epilogue<kNormedG16>(a, epilogue, s);
  if (g_dtype == kF32) return launch_epilogue<kNormedG32>(a, epilogue, s);
  return fail("gemm_skinny_normed: unknown norm scale dtype %d", g_dtype);
}

// The query/key/value product of a decode step with rotary positions and the cache write in its
// epilogue.  x: bfloat16 [m, k] (g null) -- with ssq_parts given it is bfloat16(residual * g) and the
// rows' scales come from the parts, as in bc4g_gemm_skinny_prenormed -- or the float residual stream
// with RMSNorm fused (g given, m <= 16).  q_out: bfloat16 [m, n_heads * head_dim], rotated, in the
// reordered head layout.
extern "C" int bc4g_gemm_skinny_qkv(const void* x, const void* g, int g_dtype, float eps, const float* ssq_parts,
                                    int ssq_blocks, int ssq_stride, const void* w, void* q_out,
                                    const int32_t* positions, const int32_t* slot_map, void* k_cache, void* v_cache,
                                    int m, int k, int n_heads, int n_kv_heads, int head_dim, int rotary_dim,
                                    float theta, int page_tokens, int write_kv, void* stream) {
  RopeKvArgs r{positions, slot_map, static_cast<bf16_t*>(k_cache), static_cast<bf16_t*>(v_cache), n_heads, n_kv_heads,
               head_dim, rotary_dim, page_tokens, write_kv,
               cache_fragment_order(true, head_dim, page_tokens) ? 1 : 0, theta};
  const int n = (n_heads + 2 * n_kv_heads) * head_dim;
  if (int e = check_common("gemm_skinny_qkv", m, g ? 16 : 64, n, k, kRopeKvBf16)) return e;
  if (int e = check_rope("gemm_skinny_qkv", r, n)) return e;
  BC4G_REQUIRE(!(g && ssq_parts), "gemm_skinny_qkv: the norm is either fused or prepared, not both");
  if (ssq_parts) {
    if (int e = check_parts("gemm_skinny_qkv", ssq_parts, ssq_blocks, ssq_stride, m, eps)) return e;
  }
  if (m == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  SkinnyArgs a = plain_args(x, w, q_out, m, n, k);
  a.g = g;
  a.m_stage = g ? ((m + 3) / 4) * 4 : 0;
  a.eps = eps;
  a.rope = r;
  a.ssq_parts = ssq_parts;
  a.ssq_blocks = ssq_blocks;
  a.ssq_stride = ssq_stride;
  if (!g) return launch<kRopeKvBf16, kPlain>(a, s);
  if (g_dtype == kBF16) return launch<kRopeKvBf16, kNormedG16>(a, s);
  if (g_dtype == kF32) return launch<kRopeKvBf16, kNormedG32>(a, s);
  return fail("gemm_skinny_qkv: unknown norm scale dtype %d", g_dtype);
}
