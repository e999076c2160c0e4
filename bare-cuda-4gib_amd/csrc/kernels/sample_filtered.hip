// Top-k / top-p sampling on the device, one workgroup a row.
//
// The law (the reference's, engine/src/sampler.cpp:63-104): weights w_i = exp((l_i - max) / T) in float; the
// tokens in the order of falling weight, lower id first among equal weights; the k likeliest are kept; of
// those, the fewest whose running sum reaches top_p times their total; the token drawn is the first of the
// kept ones at which u times their total minus the running sum turns negative.
//
// No sort.  A float weight's bit pattern rises with its value, so each of the three questions -- where does
// the count reach k, where does the running sum reach top_p of the total, where does it pass u of the kept
// mass -- is a walk down the patterns' digits: a histogram over the top 8 bits (the exponent) of the tokens
// in question, the bucket in which the answer lies, then the next 8 bits of that bucket's tokens, and so on
// over four levels to one exact pattern; tokens that share it are told apart by id.  A bucket's mass is kept
// as the integer sum of its tokens' mantissas (below the exponent level all tokens of a bucket share the
// exponent, and at that level a bucket is an exponent), added with integer atomics: exact, and the same in
// every run whatever order the adds arrive in.  The sums over buckets are doubles added from the top down in a
// fixed order.  (Sums in another order than the host's one-by-one walk over a sorted list: a boundary may move
// by one token when u falls within rounding of it.)
//
// A CU takes 64 lanes' instructions a clock, so what a row costs is the number of passes over its tokens times
// the instructions a token takes in each.  A first look at the exponents alone tells in which bucket the first
// question's answer lies; the tokens from that bucket up -- for a model's peaked rows a few dozen -- are copied,
// in the order of their ids, into a list in LDS (up to 18,432), and every walk runs over the list: three passes
// over the row (the maximum, the look, the list).  A flatter row's walks go over all its tokens, their patterns
// kept in LDS where the vocabulary fits (up to 36,864 tokens) and worked out again from the logits where not.
// (64 rows of 32,000 tokens: 50-64 us; of 128,256: 125-140 us, and 490 where rows are so flat that no list holds
// their candidates.  Rows run beside each other, a CU each.  On the host the same takes a download and a sort of
// the vocabulary for every row, milliseconds each, and holds the next step back until it is done.)
#include <float.h>
#include <math.h>

#include <mutex>

#include "api.h"
#include "common.h"

namespace bc4g {
namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / kWave;
constexpr int kBuckets = 256;
constexpr int kMaxCached = 36864;            // tokens whose patterns fit LDS beside the histogram (144 KB)
constexpr int kMaxListed = kMaxCached / 2;   // ... or this many (pattern, id) pairs
// A bucket's count rides in the top bits of its mantissa sum, one atomic add for both, where the vocabulary
// leaves room: 2^19 tokens of 24-bit mantissas sum to less than 2^43.
constexpr int kCountShift = 44;
constexpr int kMaxPacked = 1 << 19;

enum { kByCount = 0, kByMassGe = 1, kByMassGt = 2 };

// A prefix of a row's tokens in the law's order.
struct Prefix {
  long long bits;   // every token whose weight's pattern is above this one (-1: every token), and
  int ties;         // this many of the tokens with exactly this pattern, lowest ids first
  double mass;      // the sum of its weights (negative: not known yet)
};

struct Shared {
  unsigned int cnt[kBuckets];
  unsigned long long msum[kBuckets];
  float red_v[kWaves];
  __align__(16) int wave_cnt[kWaves];
  // a walk's state: the wave that walks a level's buckets writes it between barriers, all read it after
  unsigned int prefix;         // the digits settled so far
  unsigned int above_count;    // tokens of the universe strictly above the bucket in question
  double above_mass;
  double target;
  double total;                // the universe's mass, where a walk had to work it out
  int done;
  int found;                   // the walk's answer: found, pattern, how many of its tokens count, how many there are
  long long res_bits;
  int res_ties;
  int res_count;
  int alone_level;             // (>= 0: the answer is the one token of the bucket settled at this level; its pattern is looked up)
  int hit;
};

__device__ inline unsigned int mantissa(unsigned int b) {
  return (b >> 23) ? ((b & 0x7fffffu) | 0x800000u) : (b & 0x7fffffu);
}
__device__ inline double scaled(unsigned long long msum, unsigned int exponent) {
  // msum * 2^(exponent - 150) (a denormal's exponent counts as 1): the power of two built from its bits, the product exact
  const long long power = static_cast<long long>(static_cast<int>(exponent ? exponent : 1u) - 150 + 1023) << 52;
  return static_cast<double>(msum) * __longlong_as_double(power);
}
__device__ inline double value_of(long long bits) {
  return static_cast<double>(__uint_as_float(static_cast<unsigned int>(bits)));
}
__device__ inline bool reached(int mode, unsigned int k, double target, unsigned int count, double mass) {
  return mode == kByCount ? count >= k : mode == kByMassGe ? mass >= target : mass > target;
}

// How many of c tokens of one weight, after `above`, it takes to reach the goal: 1 .. c.
__device__ int ties_needed(int mode, unsigned int k, double target, unsigned int above_count, double above_mass,
                           double val, int c) {
  int r;
  if (mode == kByCount) {
    r = static_cast<int>(k - above_count);
  } else {
    if (!(val > 0.0)) return reached(mode, k, target, 0, above_mass) ? 1 : c;
    double need = (target - above_mass) / val;
    need = need < 0.0 ? 0.0 : need > static_cast<double>(c) ? static_cast<double>(c) : need;
    r = mode == kByMassGe ? static_cast<int>(ceil(need)) : static_cast<int>(floor(need)) + 1;
    r = r < 1 ? 1 : r > c ? c : r;
    for (int turn = 0; turn < 4 && r > 1 && reached(mode, k, target, 0, above_mass + (r - 1) * val); ++turn) --r;
    for (int turn = 0; turn < 4 && r < c && !reached(mode, k, target, 0, above_mass + r * val); ++turn) ++r;
  }
  return r < 1 ? 1 : r > c ? c : r;
}

// The tokens a walk looks at: the whole row -- patterns from LDS or from the logits -- or a list of some of them.
struct Row {
  const float* logits;
  const unsigned int* cached;    // the patterns of all tokens in LDS (null: worked out from the logits)
  const unsigned int* listed;    // (not null: the patterns of the n listed tokens, ids rising, and
  const int* listed_id;          //  their ids)
  int n;
  float row_max, inv_t;
  __device__ unsigned int bits_at(int i) const {
    if (listed) return listed[i];
    return cached ? cached[i] : __float_as_uint(expf((logits[i] - row_max) * inv_t));
  }
  __device__ int id_at(int i) const { return listed ? listed_id[i] : i; }
};

// f(pattern, index) for every token of the row that is this thread's (every kThreads-th).  From the logits, eight
// loads are on their way together: a load from memory takes hundreds of clocks, and four waves a SIMD hide few.
template <typename F>
__device__ inline void each_token(const Row& row, F f) {
  constexpr int kAhead = 8;
  if (row.listed || row.cached) {
    const unsigned int* from = row.listed ? row.listed : row.cached;
    for (int base = threadIdx.x; base < row.n; base += kAhead * kThreads) {
      unsigned int b[kAhead];
#pragma unroll
      for (int j = 0; j < kAhead; ++j) b[j] = base + j * kThreads < row.n ? from[base + j * kThreads] : 0u;
#pragma unroll
      for (int j = 0; j < kAhead; ++j)
        if (base + j * kThreads < row.n) f(b[j], base + j * kThreads);
    }
    return;
  }
  for (int base = threadIdx.x; base < row.n; base += kAhead * kThreads) {
    float l[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) l[j] = base + j * kThreads < row.n ? row.logits[base + j * kThreads] : 0.f;
#pragma unroll
    for (int j = 0; j < kAhead; ++j)
      if (base + j * kThreads < row.n) f(__float_as_uint(expf((l[j] - row.row_max) * row.inv_t)), base + j * kThreads);
  }
}

__device__ inline unsigned int wave_scan_u32(unsigned int v, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const unsigned int up = __shfl_up(v, off, kWave);
    if (lane >= off) v += up;
  }
  return v;
}
__device__ inline double wave_scan_f64(double v, int lane) {
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const double up = __shfl_up(v, off, kWave);
    if (lane >= off) v += up;
  }
  return v;
}

// Walks `universe` (those of the row's tokens that belong to it) in the law's order until the goal is reached: a
// count of k tokens, or a running sum that reaches (kByMassGe) or passes (kByMassGt) a target -- `goal` itself, or
// that fraction of the universe's mass where `of_total` (the mass is then left in sh.total).  Leaves in sh: found
// (0: the universe ends first), res_bits / res_ties (the prefix that reaches the goal ends with the res_ties-th of
// the res_count tokens of this pattern), above_count / above_mass (what lies above that pattern).  With `levels`
// below 4 the walk stops after so many digits: sh.prefix is then the bucket the answer lies in, res_count how
// many tokens it holds, above_* what lies above the bucket.  Every thread of the workgroup calls it.
//
// A level's buckets are walked by one wave, four buckets a lane from the top down: every lane adds up its own,
// a running sum over the lanes gives each what lies above it, and the first lane in which the goal is reached
// settles the bucket.
__device__ void walk(Shared& sh, const Row& row, const Prefix& universe, int mode, unsigned int k, double goal,
                     bool of_total, int levels = 4) {
  constexpr int kShift[4] = {23, 15, 7, 0};
  constexpr unsigned int kMask[4] = {0xffu, 0xffu, 0xffu, 0x7fu};
  constexpr int kPerLane = kBuckets / kWave;
  const int tid = threadIdx.x, lane = tid % kWave;
  const bool packed = row.n <= kMaxPacked;
  if (tid == 0) {
    sh.prefix = 0;
    sh.above_count = 0;
    sh.above_mass = 0.0;
    sh.done = 0;
    sh.found = 0;
    sh.alone_level = -1;
  }
  for (int level = 0; level < levels; ++level) {
    for (int i = tid; i < kBuckets; i += kThreads) {
      sh.cnt[i] = 0;
      sh.msum[i] = 0;
    }
    __syncthreads();
    const unsigned int prefix = sh.prefix;
    // a thread's tokens in a row that fall into one bucket are added as one (most of a row shares few exponents)
    int cur = -1;
    unsigned int run_count = 0;
    unsigned long long run_sum = 0;
    auto add_run = [&](int bucket) {
      if (packed) {
        atomicAdd(&sh.msum[bucket], (static_cast<unsigned long long>(run_count) << kCountShift) + run_sum);
      } else {
        atomicAdd(&sh.cnt[bucket], run_count);
        atomicAdd(&sh.msum[bucket], run_sum);
      }
    };
    const bool bounded = universe.bits >= 0;
    const unsigned int floor_bits = static_cast<unsigned int>(universe.bits);
    each_token(row, [&](unsigned int b, int) {
      if (bounded && b <= floor_bits) return;
      if (level > 0 && (b >> kShift[level - 1]) != prefix) return;
      const int bucket = static_cast<int>((b >> kShift[level]) & kMask[level]);
      if (bucket != cur) {
        if (cur >= 0) add_run(cur);
        cur = bucket, run_count = 0, run_sum = 0;
      }
      ++run_count;
      run_sum += mantissa(b);
    });
    if (cur >= 0) add_run(cur);
    __syncthreads();
    if (tid < kWave) {
      const unsigned int exponent = level == 0 ? 0u : prefix >> (23 - kShift[level - 1]);
      const int top = static_cast<int>(kMask[level]);
      unsigned int c[kPerLane];
      double m[kPerLane];
      unsigned int lane_count = 0;
      double lane_mass = 0.0;
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) {
        const int b = top - (lane * kPerLane + j);
        const unsigned long long sum = b >= 0 ? sh.msum[b] : 0ull;
        c[j] = packed ? static_cast<unsigned int>(sum >> kCountShift) : b >= 0 ? sh.cnt[b] : 0u;
        m[j] = c[j] ? scaled(packed ? sum & ((1ull << kCountShift) - 1ull) : sum, level == 0 ? static_cast<unsigned int>(b) : exponent)
                    : 0.0;
        lane_count += c[j];
        lane_mass += m[j];
      }
      const unsigned int with_count = wave_scan_u32(lane_count, lane);
      const double with_mass = wave_scan_f64(lane_mass, lane);
      const unsigned int others_count = __shfl_up(with_count, 1, kWave);
      const double others_mass = __shfl_up(with_mass, 1, kWave);
      double target = sh.target;
      if (level == 0) {
        target = goal;
        if (of_total) {
          double total = __shfl(with_mass, kWave - 1, kWave);
          if (universe.ties > 0) total += universe.ties * value_of(universe.bits);
          target = goal * total;
          if (lane == 0) sh.total = total;
        }
        if (lane == 0) sh.target = target;
      }
      unsigned int above_count = sh.above_count + (lane ? others_count : 0u);
      double above_mass = sh.above_mass + (lane ? others_mass : 0.0);
      // in this lane's buckets: the first in which the goal is reached, and the last that holds anything
      int chosen = -1, last = -1;
      unsigned int last_count = above_count;
      double last_mass = above_mass;
#pragma unroll
      for (int j = 0; j < kPerLane; ++j) {
        if (!c[j] || chosen >= 0) continue;
        last = j, last_count = above_count, last_mass = above_mass;
        if (reached(mode, k, target, above_count + c[j], above_mass + m[j])) {
          chosen = j;
        } else {
          above_count += c[j];
          above_mass += m[j];
        }
      }
      const unsigned long long crossing = __ballot(chosen >= 0), holding = __ballot(last >= 0);
      int settler = -1;                     // the lane that settles this level, and its bucket
      if (crossing != 0ull) {
        settler = __ffsll(static_cast<long long>(crossing)) - 1;
      } else if (level > 0 && holding != 0ull) {
        // the bucket as a whole reached the goal and its parts one by one fall a rounding short: its last token does
        settler = 63 - __clzll(static_cast<long long>(holding));
        chosen = last, above_count = last_count, above_mass = last_mass;
      }
      if (settler < 0) {
        // the universe's own tokens are through; it may end with some of the tokens of one more pattern
        if (lane == kWave - 1) {
          sh.above_count = above_count;
          sh.above_mass = above_mass;
          sh.done = 1;
          if (universe.ties > 0) {
            const double val = value_of(universe.bits);
            if (reached(mode, k, target, above_count + universe.ties, above_mass + universe.ties * val)) {
              sh.found = 1;
              sh.res_bits = universe.bits;
              sh.res_count = 0;            // (how many tokens there are of this pattern is not known here)
              sh.res_ties = ties_needed(mode, k, target, above_count, above_mass, val, universe.ties);
            }
          }
        }
      } else if (lane == settler) {
        const unsigned int bucket = static_cast<unsigned int>(top - (lane * kPerLane + chosen));
        const unsigned int settled = level == 0 ? bucket : (prefix << (kShift[level - 1] - kShift[level])) | bucket;
        const int count = static_cast<int>(c[chosen]);
        sh.prefix = settled;
        sh.above_count = above_count;
        sh.above_mass = above_mass;
        sh.res_count = count;
        if (level == levels - 1) {
          sh.done = 1;
          sh.found = 1;
          if (level == 3) {
            sh.res_bits = settled;
            sh.res_ties = ties_needed(mode, k, target, above_count, above_mass, value_of(settled), count);
          }
        } else if (count == 1 && levels == 4) {
          // one token in the bucket: it is the answer, whatever its other digits are
          sh.done = 1;
          sh.found = 1;
          sh.res_ties = 1;
          sh.alone_level = level;
        }
      }
    }
    __syncthreads();
    if (sh.done) break;
  }
  const int alone_level = sh.alone_level;
  if (alone_level >= 0) {
    const unsigned int digits = sh.prefix;
    const bool bounded = universe.bits >= 0;
    const unsigned int floor_bits = static_cast<unsigned int>(universe.bits);
    each_token(row, [&](unsigned int b, int) {
      if ((!bounded || b > floor_bits) && (b >> kShift[alone_level]) == digits) sh.res_bits = b;
    });
    __syncthreads();
  }
}

// Where this thread's `mine` items go among those of all the workgroup's threads, in the order of the threads, and
// how many there are of all.  Every thread calls it (two barriers).
__device__ inline void place_among(Shared& sh, unsigned int mine, int& place, int& all) {
  static_assert(kWaves == 16, "the waves' counts are read as four int4");
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const unsigned int with_mine = wave_scan_u32(mine, lane);
  if (lane == kWave - 1) sh.wave_cnt[wave] = static_cast<int>(with_mine);
  __syncthreads();
  int before = 0;
  all = 0;
#pragma unroll
  for (int q = 0; q < kWaves / 4; ++q) {
    const int4 c = reinterpret_cast<const int4*>(sh.wave_cnt)[q];
    before += (4 * q < wave ? c.x : 0) + (4 * q + 1 < wave ? c.y : 0) + (4 * q + 2 < wave ? c.z : 0) + (4 * q + 3 < wave ? c.w : 0);
    all += c.x + c.y + c.z + c.w;
  }
  place = before + static_cast<int>(with_mine - mine);
  __syncthreads();
}

// The id of the r-th of the `count` tokens, in the order of the ids, whose weight has this pattern; into sh.hit.
__device__ void locate(Shared& sh, const Row& row, unsigned int bits, int r, int count) {
  if (count == 1) {                                     // the one there is: nothing to put in order
    each_token(row, [&](unsigned int b, int i) {
      if (b == bits) sh.hit = row.id_at(i);
    });
    return;
  }
  int seen = 0;
  for (int base = 0; base < row.n; base += kThreads) {
    const int i = base + threadIdx.x;
    const bool match = i < row.n && row.bits_at(i) == bits;
    int place, all;
    place_among(sh, match ? 1u : 0u, place, all);
    if (match && seen + place + 1 == r) sh.hit = row.id_at(i);
    seen += all;
    if (seen >= r) break;
  }
}

// The row's tokens whose pattern is `bound` or above, in the order of their ids, into the list; how many.
// The row is one whose patterns come from the logits.  Eight tokens in a row to a thread and turn; a turn's
// logits are asked for a turn ahead, so that the way from memory lies beside the turn before's barriers.
__device__ int list_from(Shared& sh, const Row& row, unsigned int bound, unsigned int* listed, int* listed_id) {
  constexpr int kEach = 8;
  auto ask = [&](int base, float (&l)[kEach]) {
    const int first = base + kEach * threadIdx.x;
#pragma unroll
    for (int j = 0; j < kEach; ++j) l[j] = first + j < row.n ? row.logits[first + j] : 0.f;
  };
  int seen = 0;
  float next[kEach];
  ask(0, next);
  for (int base = 0; base < row.n; base += kEach * kThreads) {
    const int first = base + kEach * threadIdx.x;
    unsigned int b[kEach];
    unsigned int mine = 0;
#pragma unroll
    for (int j = 0; j < kEach; ++j) {
      b[j] = __float_as_uint(expf((next[j] - row.row_max) * row.inv_t));
      mine += first + j < row.n && b[j] >= bound ? 1u : 0u;
    }
    if (base + kEach * kThreads < row.n) ask(base + kEach * kThreads, next);
    int place, all;
    place_among(sh, mine, place, all);
    int at = seen + place;
#pragma unroll
    for (int j = 0; j < kEach; ++j) {
      if (first + j < row.n && b[j] >= bound) {
        listed[at] = b[j];
        listed_id[at] = first + j;
        ++at;
      }
    }
    seen += all;
  }
  __syncthreads();
  return seen;
}

__global__ __launch_bounds__(kThreads) void sample_filtered_kernel(
    const float* __restrict__ logits, const int32_t* __restrict__ rows, const float* __restrict__ temperature,
    const double* __restrict__ u, const int32_t* __restrict__ top_k, const double* __restrict__ top_p,
    int32_t* __restrict__ out, int vocab, int cache_patterns) {
  __shared__ Shared sh;
  extern __shared__ unsigned int room[];            // the row's patterns, or the list's patterns and ids
  const int which = blockIdx.x;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  Row whole;
  whole.logits = logits + static_cast<size_t>(rows[which]) * vocab;
  whole.cached = nullptr;
  whole.listed = nullptr;
  whole.listed_id = nullptr;
  whole.n = vocab;

  float v = -FLT_MAX;
  for (int base = threadIdx.x; base < vocab; base += 8 * kThreads) {
    float l[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) l[j] = base + j * kThreads < vocab ? whole.logits[base + j * kThreads] : -FLT_MAX;
#pragma unroll
    for (int j = 0; j < 8; ++j) v = fmaxf(v, l[j]);
  }
  v = wave_max(v);
  if (lane == 0) sh.red_v[wave] = v;
  __syncthreads();
  v = sh.red_v[0];
  for (int w = 1; w < kWaves; ++w) v = fmaxf(v, sh.red_v[w]);
  whole.row_max = v;
  whole.inv_t = 1.0f / temperature[which];
  if (threadIdx.x == 0) sh.hit = 0;
  __syncthreads();

  const unsigned int k = top_k[which] > 0 && top_k[which] < vocab ? static_cast<unsigned int>(top_k[which])
                                                                 : static_cast<unsigned int>(vocab);
  const bool count_first = k < static_cast<unsigned int>(vocab);
  const double p = top_p[which];
  const Prefix everything = {-1, 0, -1.0};
  Prefix kept = everything;
  Row row = whole;
  {
    // a look at the exponents alone: the bucket in which the first question's answer lies, and how many tokens
    // there are from that bucket up -- if the list holds them, they are all that the walks have to look at
    if (count_first) walk(sh, whole, everything, kByCount, k, 0.0, false, 1);
    else walk(sh, whole, everything, kByMassGe, 0, p, true, 1);
    const bool found = sh.found;
    const unsigned int bucket = sh.prefix, candidates = sh.above_count + static_cast<unsigned int>(sh.res_count);
    if (!count_first) kept.mass = sh.total;
    __syncthreads();
    if (found && candidates <= static_cast<unsigned int>(kMaxListed)) {
      int* listed_id = reinterpret_cast<int*>(room + kMaxListed);
      row.n = list_from(sh, whole, bucket << 23, room, listed_id);
      row.listed = room;
      row.listed_id = listed_id;
    } else if (cache_patterns) {
      for (int i = threadIdx.x; i < vocab; i += kThreads) room[i] = whole.bits_at(i);
      __syncthreads();
      whole.cached = room;
      row = whole;
    }
  }
  // the k likeliest
  if (count_first) {
    walk(sh, row, everything, kByCount, k, 0.0, false);
    if (sh.found) kept = {sh.res_bits, sh.res_ties, sh.above_mass + sh.res_ties * value_of(sh.res_bits)};
    __syncthreads();
  }
  // of those, the fewest that reach top_p of their total
  Prefix nucleus = kept;
  if (p < 1.0) {
    const bool of_total = kept.mass < 0.0;
    walk(sh, row, kept, kByMassGe, 0, of_total ? p : p * kept.mass, of_total);
    if (sh.found) nucleus = {sh.res_bits, sh.res_ties, sh.above_mass + sh.res_ties * value_of(sh.res_bits)};
    else if (of_total) nucleus.mass = sh.total;       // (rounding left the sum a hair short: everything is kept)
    __syncthreads();
  }
  // the first of those at which the running sum passes u of their mass
  const bool of_total = nucleus.mass < 0.0;
  walk(sh, row, nucleus, kByMassGt, 0, of_total ? u[which] : u[which] * nucleus.mass, of_total);
  long long bits = sh.res_bits;
  int r = sh.res_ties, count = sh.res_count;
  const bool found = sh.found;
  __syncthreads();
  if (!found) {                                        // rounding again: the last of the kept tokens
    if (nucleus.bits >= 0 && nucleus.ties > 0) {
      bits = nucleus.bits, r = nucleus.ties, count = 0;            // (how many there are of it is not known here)
    } else {
      row = whole;
      walk(sh, row, everything, kByCount, static_cast<unsigned int>(vocab), 0.0, false);
      bits = sh.res_bits, r = sh.res_ties, count = sh.res_count;
      __syncthreads();
    }
  }
  locate(sh, row, static_cast<unsigned int>(bits), r, count);
  __syncthreads();
  if (threadIdx.x == 0) out[rows[which]] = sh.hit;
}

}  // namespace
}  // namespace bc4g

using namespace bc4g;

// For each of n rows: draws the token of logits row rows[i] by the law above with temperature[i] (> 0), the
// uniform number u[i] in [0, 1), top_k[i] (0 or >= vocab: no limit) and top_p[i] (>= 1: no limit), into
// out[rows[i]].  logits: float [*, vocab], contiguous.
extern "C" int bc4g_sample_filtered(const float* logits, const int32_t* rows, const float* temperature, const double* u,
                                    const int32_t* top_k, const double* top_p, int32_t* out, int n, int vocab,
                                    void* stream) {
  BC4G_REQUIRE(n >= 0 && vocab > 0, "sample_filtered: bad sizes rows=%d V=%d", n, vocab);
  if (n == 0) return 0;
  const int cache_patterns = vocab <= kMaxCached ? 1 : 0;
  const size_t lds = static_cast<size_t>(kMaxCached) * sizeof(unsigned int);      // the list's room, or the patterns'
  static std::once_flag once;
  static hipError_t raised = hipSuccess;
  std::call_once(once, [] {
    raised = hipFuncSetAttribute(reinterpret_cast<const void*>(sample_filtered_kernel),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, kMaxCached * sizeof(unsigned int));
  });
  if (raised != hipSuccess) return fail("sample_filtered: cannot raise the dynamic LDS limit to %d bytes",
                                        static_cast<int>(kMaxCached * sizeof(unsigned int)));
  sample_filtered_kernel<<<n, kThreads, lds, static_cast<hipStream_t>(stream)>>>(logits, rows, temperature, u, top_k,
                                                                               top_p, out, vocab, cache_patterns);
  return check_launch("sample_filtered");
}
