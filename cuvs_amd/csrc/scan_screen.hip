/*
 * Screening pass of the L2 early stop (8-bit codes; 4-bit codes through the table-free kernel).
 *
 * A row's score is a sum of non-negative table entries taken in subspace order, so the partial sum
 * over the first S subspaces is a lower bound of its final score, and it is exactly the
 * intermediate value the full scan kernels reach after S additions.  A pair none of whose rows is
 * still at or below the query's current k-th best score after those S terms cannot contribute a
 * result (compute_score's early stop in the reference,
 * cpp/src/neighbors/ivf_pq/detail/jit_lto_kernels/compute_score_impl.cuh:70-74, applied to the whole
 * list at once).  For clustered data this removes most (query, probe) pairs for an eighth of the
 * table-building and gather work, and only the survivors go through the full scan.  S = 8 by
 * default (the first half of each row's first 16-byte chunk): on the benchmark data as many pairs
 * are dropped as with 16, and with 4 three times as many survive.  The same 8 bytes of a row of
 * 4-bit codes hold 16 subspaces of 16 entries.
 *
 * Organisation: persistent 256-thread blocks, several per CU so that the table-building phase of
 * one block overlaps the gather phase of another.  A block takes G = 4 pairs per iteration; thread
 * c keeps entry c of the first S subspaces' codebooks in registers and builds entry c of the four
 * S x 256 tables; then wave g sums the first S codes of every row of pair g and stops at the first
 * tile with a row still in play.
 */
#include "device_utils.cuh"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstddef>
#include <cstdlib>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

#define LDS_AS __attribute__((address_space(3)))
#define GLOBAL_AS __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

/** Leading codes of a row: 8 bytes when the screen sums at most 8 subspaces, else the 16-byte chunk. */
template <int SUBS>
struct screen_codes {
  using type = typename std::conditional<(SUBS <= 8), u32x2, u32x4>::type;
};

constexpr uint32_t kScreenThreads = 256;
constexpr uint32_t kScreenG       = 4;   // pairs per block iteration = waves per block
constexpr uint32_t kScreenLdsBase = 16;  // no LDS object at address 0: a null constant pointer folds badly

__device__ __forceinline__ void lds_barrier_s()
{
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ float opaque_one_s()
{
  float one = 1.0f;
  asm volatile("" : "+v"(one));
  return one;
}

/*
 * Surviving pairs are appended to one list shared by the whole grid.  One atomic add per pair on
 * its counter would serialise every wave of the grid on a single address (about 11 ns per add,
 * which bounds the kernel as soon as most pairs survive), so a wave collects up to
 * kSurvivorBatch records in an LDS area of its own and claims their slots with one add.
 * A record is 8 dwords: a full batch is four dwords per lane.
 */
constexpr uint32_t kSurvivorBatch      = 32;
constexpr uint32_t kSurvivorBatchBytes = kSurvivorBatch * uint32_t(sizeof(pair_desc));
static_assert(kSurvivorBatchBytes == 4 * 64 * 4, "a full batch is four dwords per lane");
static_assert(offsetof(pair_desc, q) == 8 && offsetof(pair_desc, row_off) == 28, "record layout");

/** Length class of a list of n_rows rows: by its number of 64-row tiles, the longest first. */
__device__ __forceinline__ uint32_t class_of_rows(uint32_t n_rows)
{
  const uint32_t tiles = (n_rows + 63u) >> 6;
  return tiles >= kSurvivorClasses ? 0u : kSurvivorClasses - 1u - tiles;
}

__device__ __forceinline__ void flush_survivors(LDS_AS uint32_t* pending, uint32_t n, uint32_t lane,
                                                pair_desc* __restrict__ survivors,
                                                uint32_t* __restrict__ n_survivors)
{
  uint32_t pos = 0;
  if (lane == 0) { pos = atomicAdd(n_survivors, n); }
  pos = uint32_t(__builtin_amdgcn_readfirstlane(pos));
  auto* dst = reinterpret_cast<uint32_t*>(survivors + pos);
  for (uint32_t w = lane; w < n * 8u; w += 64u) { dst[w] = pending[w]; }
}

/** Adds a record to the wave's batch (all lanes call it; `n` is the same in all of them). */
__device__ __forceinline__ void push_survivor(LDS_AS uint32_t* pending, uint32_t& n, uint32_t lane,
                                              const pair_desc& d, pair_desc* __restrict__ survivors,
                                              uint32_t* __restrict__ n_survivors,
                                              uint8_t* __restrict__ alive)
{
  if (lane == 0) {
    // the record's eight dwords in memory order
    const uint64_t ptr   = reinterpret_cast<uint64_t>(d.data);
    LDS_AS uint32_t* dst = pending + n * 8u;
    dst[0]               = uint32_t(ptr);
    dst[1]               = uint32_t(ptr >> 32);
    dst[2]               = d.q;
    dst[3]               = d.slot;
    dst[4]               = d.label;
    dst[5]               = d.sample_off;
    dst[6]               = d.n_rows;
    dst[7]               = d.row_off;
    alive[d.slot]        = 1;
  }
  n++;
  if (n == kSurvivorBatch) {
    flush_survivors(pending, n, lane, survivors, n_survivors);
    n = 0;
  }
}

/** Leading subspaces the table-building screen sums (of the 16 in the first chunk): with 16 the
 *  same pairs survive on clustered data, with 4 three times as many. */
constexpr int kScreenSubs = 8;
/** The table-free screen checks for the first time after this many subspaces, then after 4 and 8. */
constexpr int kScreenFirstCheck = 2;

template <int SUBS, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER>
__global__ __launch_bounds__(kScreenThreads, 4) void scan_screen_kernel(
  scan_args a, const pair_desc* __restrict__ desc, uint32_t n_pairs, uint32_t group_bytes,
  pair_desc* __restrict__ survivors, uint32_t* __restrict__ n_survivors, uint8_t* __restrict__ alive)
{
  using traits = lut_traits<LUT>;
  using lut_t  = typename traits::storage;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  using codes_t = typename screen_codes<SUBS>::type;
  constexpr uint32_t G           = kScreenG;
  constexpr uint32_t SUB         = SUBS;
  constexpr uint32_t NDIFF       = SUB * PQ_LEN;  // leading rotated dimensions the first chunk covers
  constexpr uint32_t lut_entries = SUB * 256u;
  constexpr uint32_t off_diff    = kScreenLdsBase + G * lut_entries * uint32_t(sizeof(lut_t));
  static_assert(G * NDIFF <= kScreenThreads, "one thread stages one (pair, dimension)");
  constexpr uint32_t off_pending = off_diff + G * NDIFF * 4u;
  auto* lut_all  = reinterpret_cast<LDS_AS lut_t*>(uintptr_t(kScreenLdsBase));
  auto* diff_all = reinterpret_cast<LDS_AS float*>(uintptr_t(off_diff));
  const float one = opaque_one_s();

  const uint32_t tid     = threadIdx.x;
  const uint32_t lane    = tid & 63u;
  const uint32_t wid     = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (a.screen_pairs_dev != nullptr) { n_pairs = uint32_t(__builtin_amdgcn_readfirstlane(*a.screen_pairs_dev)); }
  const uint32_t n_iters = (n_pairs + G - 1u) / G;
  const uint32_t stride  = gridDim.x;
  if (blockIdx.x >= n_iters) { return; }
  auto* my_lut = lut_all + wid * lut_entries;
  auto* pending = reinterpret_cast<LDS_AS uint32_t*>(uintptr_t(off_pending + wid * kSurvivorBatchBytes));
  uint32_t n_pending = 0;

  float book[PER_CLUSTER ? 1 : SUB][PQ_LEN];
  if (!PER_CLUSTER) {
#pragma unroll
    for (uint32_t j = 0; j < SUB; j++) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) { book[j][t] = a.pq_centers[(j * PQ_LEN + t) * 256 + tid]; }
    }
  }

  auto record = [&](uint32_t it, uint32_t g) -> pair_desc {
    const uint32_t slot = it * G + g;
    pair_desc d         = desc[slot < n_pairs ? slot : n_pairs - 1u];
    if (slot >= n_pairs) { d.n_rows = 0; d.slot = 0xFFFFFFFFu; }
    return d;
  };
  // the record a wave scans is the same in all its lanes: say so, and the tile loop's trip count,
  // addresses and bound stay in scalar registers
  auto uniform = [](pair_desc d) -> pair_desc {
    const uint64_t p = reinterpret_cast<uint64_t>(d.data);
    // the builtin returns a signed int: widen through uint32_t, or the low half sign-extends
    const uint32_t hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p >> 32)));
    const uint32_t lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(p)));
    const uint64_t u  = (uint64_t(hi) << 32) | uint64_t(lo);
    d.data       = reinterpret_cast<const uint8_t*>(u);
    d.q          = uint32_t(__builtin_amdgcn_readfirstlane(d.q));
    d.slot       = uint32_t(__builtin_amdgcn_readfirstlane(d.slot));
    d.n_rows     = uint32_t(__builtin_amdgcn_readfirstlane(d.n_rows));
    d.row_off    = uint32_t(__builtin_amdgcn_readfirstlane(d.row_off));
    return d;
  };
  // first chunk of row (64 * tile + lane) of a list; the code arena carries two groups of slack
  // after the last list, so whole tiles can be read without clamping the row
  const uint32_t lane_off = (lane >> 5) * group_bytes + (lane & 31u) * 16u;
  auto chunk_ptr = [&](const uint8_t* list_data, uint32_t tile) {
    return reinterpret_cast<const GLOBAL_AS codes_t*>(reinterpret_cast<uintptr_t>(list_data) +
                                                      uint64_t(tile) * (2u * group_bytes) + lane_off);
  };
  // Where the index keeps the plane of leading codes, a tile's eight leading bytes a row are one
  // contiguous 512-byte load (from the interleaved lists: every other 8 bytes of two groups), and
  // the plane's slack lets a wave request tiles unconditionally, two ahead of the one it sums.
  const bool use_plane = SUBS <= 8 && a.lead_plane != nullptr;  // uniform
  auto codes_of = [&](const pair_desc& d, uint32_t tile) -> codes_t {
    if constexpr (SUBS <= 8) {
      if (use_plane) {
        const auto* plane = reinterpret_cast<const GLOBAL_AS u32x2*>(reinterpret_cast<uintptr_t>(a.lead_plane));
        return plane[uint64_t(d.row_off) + tile * 64u + lane];
      }
    }
    return *chunk_ptr(d.data, tile);
  };
  // staging element (pair tid / NDIFF, dimension tid % NDIFF) of iteration `it`
  auto fetch_diff = [&](uint32_t it) -> float {
    float v = 0.0f;
    if (tid < G * NDIFF) {
      const pair_desc d = record(it, tid / NDIFF);
      if (d.n_rows != 0) {
        v = a.rot_q[uint64_t(d.q) * a.rot_dim + tid % NDIFF] -
            a.centers_rot[uint64_t(d.label) * a.rot_dim + tid % NDIFF];
      }
    }
    return v;
  };

  uint32_t it   = blockIdx.x;
  float staged  = fetch_diff(it);
  pair_desc my_d = uniform(record(it, wid));
  codes_t cur{}, cur1{};
  uint32_t thr   = 0xFFFFFFFFu;
  if (my_d.n_rows != 0) {
    cur = codes_of(my_d, 0u);
    if (use_plane) { cur1 = codes_of(my_d, 1u); }
    thr = uint32_t(__builtin_amdgcn_readfirstlane(a.query_kth[my_d.q]));
  }
  if (tid < G * NDIFF) { diff_all[tid] = staged; }
  lds_barrier_s();

  for (;;) {
    const bool has_next    = it + stride < n_iters;
    const uint32_t nxt_it  = has_next ? it + stride : it;
    if (has_next) { staged = fetch_diff(nxt_it); }
    const pair_desc nxt_d = uniform(record(nxt_it, wid));

    /* ---- the G tables of the first chunk, entry `tid` of each subspace ---- */
#pragma unroll
    for (uint32_t g = 0; g < G; g++) {
      const pair_desc dg = record(it, g);
      if (dg.n_rows == 0) { continue; }  // uniform
      float cb[PQ_LEN];
      if (PER_CLUSTER) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) { cb[t] = a.pq_centers[(uint64_t(dg.label) * PQ_LEN + t) * 256 + tid]; }
      }
      const auto* diff = diff_all + g * NDIFF;
      auto* lut        = lut_all + g * lut_entries;
#pragma unroll
      for (uint32_t j = 0; j < SUB; j++) {
        float score = 0.0f;
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          const float pqc = PER_CLUSTER ? cb[t] : book[PER_CLUSTER ? 0 : j][t];
          float df        = diff[j * PQ_LEN + t];
          df -= pqc;
          score = fmaf(df, df, score);
        }
        lut[j * 256 + tid] = traits::encode(score);
      }
    }
    lds_barrier_s();  // tables complete; the staged terms are free again
    if (has_next && tid < G * NDIFF) { diff_all[tid] = staged; }

    /* ---- wave `wid` sums the first chunk of every row of its pair ---- */
    if (my_d.slot != 0xFFFFFFFFu) {
      const uint32_t n_rows    = my_d.n_rows;
      const uint32_t n_tiles   = (n_rows + 63u) >> 6;
      const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
      bool in_play             = false;
      // sums the leading codes `c8` of the rows of tile `tile`
      auto sum_tile = [&](const codes_t& c8, uint32_t tile) __attribute__((always_inline)) {
        const uint32_t i = tile * 64u + lane;
        uint32_t w[4] = {c8.x, c8.y, 0u, 0u};
        if constexpr (SUBS > 8) {
          w[2] = c8.z;
          w[3] = c8.w;
        }
        acc_t acc           = acc_t(0);
        auto add_codes = [&](int first, int last) __attribute__((always_inline)) {
#pragma unroll
          for (int kk = first; kk < last; kk++) {
            const uint32_t c = (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu;
            const lut_t v    = my_lut[kk * 256 + c];
            if (OUT_HALF) {
              acc = acc_t(acc + traits::to_half(v));
            } else if (LUT == LUT_F16) {
              acc = acc_t(fmaf(traits::to_float(v), one, float(acc)));
            } else {
              acc = acc_t(acc + traits::to_float(v));
            }
          }
        };
        // most tiles are decided by half of the screening subspaces already
        add_codes(0, SUBS / 2);
        in_play = __ballot(i < n_rows && !(__float_as_uint(float(acc)) > stop_bits)) != 0ull;
        if (in_play) {
          add_codes(SUBS / 2, SUBS);
          in_play = __ballot(i < n_rows && !(__float_as_uint(float(acc)) > stop_bits)) != 0ull;
        }
      };
      if (use_plane) {
        // three registers take turns: two tiles are in flight while one is summed
        codes_t r0 = cur, r1 = cur1, r2;
        for (uint32_t tile = 0; tile < n_tiles; tile += 3u) {
          r2 = codes_of(my_d, tile + 2u);
          sum_tile(r0, tile);
          if (in_play || tile + 1u >= n_tiles) { break; }
          r0 = codes_of(my_d, tile + 3u);
          sum_tile(r1, tile + 1u);
          if (in_play || tile + 2u >= n_tiles) { break; }
          r1 = codes_of(my_d, tile + 4u);
          sum_tile(r2, tile + 2u);
          if (in_play) { break; }
        }
      } else {
        for (uint32_t tile = 0; tile < n_tiles && !in_play; tile++) {
          codes_t ahead = cur;
          if (tile + 1u < n_tiles) { ahead = *chunk_ptr(my_d.data, tile + 1u); }
          sum_tile(cur, tile);
          cur = ahead;
        }
      }
      if (in_play) { push_survivor(pending, n_pending, lane, my_d, survivors, n_survivors, alive); }
    }

    if (!has_next) { break; }
    my_d = nxt_d;
    thr  = 0xFFFFFFFFu;
    if (my_d.n_rows != 0) {
      cur = codes_of(my_d, 0u);
      if (use_plane) { cur1 = codes_of(my_d, 1u); }
      thr = uint32_t(__builtin_amdgcn_readfirstlane(a.query_kth[my_d.q]));
    }
    it = nxt_it;
    lds_barrier_s();  // every wave is done with the tables; next staged terms are visible
  }
  if (n_pending != 0) { flush_survivors(pending, n_pending, lane, survivors, n_survivors); }
}

/*
 * Screening without tables, for per-subspace codebooks.
 *
 * A list of the benchmark index has a few hundred rows, and most tiles of 64 rows are decided by
 * their first two to four codes: a 256-entry table per subspace would be built for about as many
 * lookups as it has entries.  Here the block keeps the first 8 subspaces' codebooks in LDS once,
 * and a lane computes the table entry its row's code selects on the spot: the same subtractions,
 * FMAs and rounding to the table's type, so the partial sums are the ones the table kernels form.
 * Only the subspaces that every tile looks at (the first FIRST) get a table of the wave's own, and
 * only for a list long enough to repay it.
 * Nothing is shared between the waves of a block after the codebooks are loaded: each wave walks
 * its own sequence of pairs, with the next pair's record, first codes, bound and query-minus-centre
 * terms in flight while it scans the current one.
 */
/** The pairs of a wave of the persistent screening kernels: pair first, first + stride, ... below
 *  end.  Workgroups go to the XCDs in turn, and pairs come in list order: the waves of one XCD take
 *  one contiguous eighth of the pairs (neighbouring waves neighbouring pairs), so that a list's
 *  leading codes pass through one XCD's L2 instead of all eight. */
struct wave_pairs {
  uint32_t first, stride, end;
};
__device__ __forceinline__ wave_pairs screen_wave_pairs(uint32_t n_pairs, uint32_t wid, uint32_t waves_per_block)
{
  const uint32_t grid = gridDim.x;
  if ((grid & 7u) == 0u && n_pairs >= grid * waves_per_block) {
    const uint32_t chunk = (n_pairs + 7u) >> 3;
    const uint32_t lo    = (blockIdx.x & 7u) * chunk;
    const uint32_t hi    = lo + chunk < n_pairs ? lo + chunk : n_pairs;
    return {lo + (blockIdx.x >> 3) * waves_per_block + wid, (grid >> 3) * waves_per_block, hi};
  }
  return {blockIdx.x * waves_per_block + wid, grid * waves_per_block, n_pairs};
}

constexpr uint32_t kDirectThreads = 512;
constexpr uint32_t kDirectSubs    = 8;
constexpr uint32_t kIpRounds      = 12;  // the inner-product screen keeps a value per 64 subspaces: pq_dim <= 768

template <int PQ_LEN>
struct book_vec;
template <>
struct book_vec<1> {
  typedef float type __attribute__((ext_vector_type(1)));
};
template <>
struct book_vec<2> {
  typedef float type __attribute__((ext_vector_type(2)));
};
template <>
struct book_vec<3> {
  typedef float type __attribute__((ext_vector_type(4)));  // the fourth component is not used
};
template <>
struct book_vec<4> {
  typedef float type __attribute__((ext_vector_type(4)));
};
template <>
struct book_vec<8> {
  typedef float type __attribute__((ext_vector_type(8)));
};

template <int PQ_LEN, int LUT, bool OUT_HALF, int FIRST, int BITS, bool PER_CLUSTER = false>
__global__ __launch_bounds__(kDirectThreads, 2) void scan_screen_direct_kernel(
  scan_args a, const pair_desc* __restrict__ desc, uint32_t n_pairs, uint32_t group_bytes,
  pair_desc* __restrict__ survivors, uint32_t* __restrict__ n_survivors, uint8_t* __restrict__ alive)
{
  using traits = lut_traits<LUT>;
  using lut_t  = typename traits::storage;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  using vec_t  = typename book_vec<PQ_LEN>::type;
  // the eight leading code bytes of a row: 8 subspaces of 256 entries, or 16 of 16 (4-bit codes)
  static_assert(BITS == 8 || BITS == 4, "byte or nibble codes");
  constexpr uint32_t SUB   = BITS == 8 ? kDirectSubs : 2u * kDirectSubs;
  constexpr uint32_t BOOK  = 1u << BITS;
  constexpr int MID        = BITS == 8 ? 4 : 8;  // the second look at the bound
  constexpr uint32_t NDIFF = SUB * PQ_LEN;
  static_assert(NDIFF <= 64, "one lane per leading rotated dimension");
  static_assert(FIRST <= 4 && FIRST <= MID, "the first subspaces' terms sit in scalar registers");
  // Per-cluster codebooks: one codebook of 256 entries a list, for all of its subspaces.  Each wave
  // keeps the codebook of its current pair's list in its own eighth of the area that otherwise
  // holds the eight leading subspaces' codebooks (the same bytes: eight waves a block), fetched a
  // pair ahead like the pair's other operands (2 KB for two dimensions a subspace, out of L2:
  // neighbouring waves work on pairs of the same list).
  static_assert(!PER_CLUSTER || (BITS == 8 && kDirectThreads / 64u == SUB), "a wave's codebook takes one subspace's place");
  constexpr uint32_t NCB = PER_CLUSTER ? BOOK / 64u : 1u;  // codebook entries a lane fetches
  auto* book      = reinterpret_cast<LDS_AS vec_t*>(uintptr_t(kScreenLdsBase));
  const float one = opaque_one_s();
  constexpr uint32_t off_pending = kScreenLdsBase + SUB * BOOK * uint32_t(sizeof(vec_t));
  constexpr uint32_t off_mini    = off_pending + (kDirectThreads / 64u) * kSurvivorBatchBytes;
  constexpr uint32_t kMiniTiles  = 6;

  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr uint32_t WPB = kDirectThreads / 64u;
  if (a.screen_pairs_dev != nullptr) { n_pairs = uint32_t(__builtin_amdgcn_readfirstlane(*a.screen_pairs_dev)); }
  const wave_pairs mine  = screen_wave_pairs(n_pairs, wid, WPB);
  const uint32_t total   = mine.stride;
  const uint32_t p_end   = mine.end;
  if (mine.first - wid >= p_end) { return; }  // the whole block, before its barrier

  if constexpr (!PER_CLUSTER) {
    for (uint32_t e = tid; e < SUB * BOOK; e += kDirectThreads) {
      vec_t v = {};
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) { v[t] = a.pq_centers[((e / BOOK) * PQ_LEN + t) * BOOK + (e % BOOK)]; }
      book[e] = v;
    }
    lds_barrier_s();
  }

  uint32_t p = mine.first;
  if (p >= p_end) { return; }
  auto* my_book = book + (PER_CLUSTER ? wid * BOOK : 0u);  // per cluster: entry `code` of the pair's list
  auto* pending = reinterpret_cast<LDS_AS uint32_t*>(uintptr_t(off_pending + wid * kSurvivorBatchBytes));
  auto* mini    = reinterpret_cast<LDS_AS lut_t*>(uintptr_t(off_mini + wid * uint32_t(FIRST) * 256u * uint32_t(sizeof(lut_t))));
  uint32_t n_pending = 0;
  uint32_t n_far     = 0;  // pairs this wave dropped on their length

  // A record is fetched two pairs ahead with a vector load (index hidden from the uniformity
  // analysis): a scalar load would be waited for by the tile loop's first LDS read, since both
  // count on the same counter, while vector loads return in order behind loads issued earlier.
  auto record = [&](uint32_t idx) -> pair_desc {
    uint32_t at = idx < p_end ? idx : p_end - 1u;
    asm volatile("" : "+v"(at));
    return desc[at];
  };
  auto uniform = [](pair_desc d) -> pair_desc {
    const uint64_t ptr = reinterpret_cast<uint64_t>(d.data);
    // the builtin returns a signed int: widen through uint32_t, or the low half sign-extends
    const uint32_t hi = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(ptr >> 32)));
    const uint32_t lo = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(ptr)));
    d.data       = reinterpret_cast<const uint8_t*>((uint64_t(hi) << 32) | uint64_t(lo));
    d.q          = uint32_t(__builtin_amdgcn_readfirstlane(d.q));
    d.slot       = uint32_t(__builtin_amdgcn_readfirstlane(d.slot));
    d.label      = uint32_t(__builtin_amdgcn_readfirstlane(d.label));
    d.sample_off = uint32_t(__builtin_amdgcn_readfirstlane(d.sample_off));
    d.n_rows     = uint32_t(__builtin_amdgcn_readfirstlane(d.n_rows));
    d.row_off    = uint32_t(__builtin_amdgcn_readfirstlane(d.row_off));
    return d;
  };
  // Codes 0..7 of row (64 * tile + lane) of a list come from the packed plane of leading codes
  // (kLeadPlaneSlack slots of slack follow the last list).
  const auto* plane = reinterpret_cast<const GLOBAL_AS u32x2*>(reinterpret_cast<uintptr_t>(a.lead_plane));
  auto lead_codes = [&](const pair_desc& d, uint32_t tile) {
    return plane[uint64_t(d.row_off) + tile * 64u + lane];
  };
  // lane d < rot_dim: (rotated query - rotated centre)[d] of a pair (0 in the lanes past rot_dim)
  const uint32_t rot_dim = a.rot_dim;
  auto fetch_diff = [&](const pair_desc& d) -> float {
    const uint32_t dim = lane < rot_dim ? lane : 0u;
    const float df = a.rot_q[uint64_t(d.q) * rot_dim + dim] - a.centers_rot[uint64_t(d.label) * rot_dim + dim];
    return lane < rot_dim ? df : 0.0f;
  };
  // The pair's whole residual, for its length: dimensions 64 + 64 x + lane as well (rot_dim up to
  // 64 (1 + kFarDims)), and the radius of its list.  A pair whose rows are all provably past the
  // query's bound is dropped before its first tile.
  constexpr uint32_t kFarDims = 3;
  const bool by_length = a.prune_keep > 0.0f && a.list_radius != nullptr && rot_dim <= 64u * (1u + kFarDims);
  struct far_part {
    float v[kFarDims];
    float radius;
  };
  auto fetch_far = [&](const pair_desc& d) -> far_part {
    far_part f{};
    if (by_length) {
#pragma unroll
      for (uint32_t x = 0; x < kFarDims; x++) {
        const uint32_t dim = 64u * (x + 1u) + lane;
        const uint32_t at  = dim < rot_dim ? dim : 0u;
        const float df = a.rot_q[uint64_t(d.q) * rot_dim + at] - a.centers_rot[uint64_t(d.label) * rot_dim + at];
        f.v[x]         = dim < rot_dim ? df : 0.0f;
      }
      f.radius = a.list_radius[d.label];
    }
    return f;
  };

  // per cluster: entries lane, lane + 64, ... of a pair's list's codebook
  struct book_part {
    vec_t v[NCB];
  };
  auto fetch_book = [&](const pair_desc& d) -> book_part {
    book_part b{};
    if constexpr (PER_CLUSTER) {
#pragma unroll
      for (uint32_t c = 0; c < NCB; c++) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) { b.v[c][t] = a.pq_centers[(uint64_t(d.label) * PQ_LEN + t) * BOOK + c * 64u + lane]; }
      }
    }
    return b;
  };

  pair_desc d0 = uniform(record(p));
  pair_desc d1 = uniform(record(p + total));
  // leading codes of a pair's tiles 0 and 1 (the plane's slack covers tiles past a list's end)
  u32x2 lead0 = lead_codes(d0, 0u);
  u32x2 next0 = lead_codes(d0, 1u);
  uint32_t thr0  = a.query_kth[d0.q];
  float dv0     = fetch_diff(d0);
  far_part far0 = fetch_far(d0);
  book_part cb0 = fetch_book(d0);

  for (;;) {
    const bool has1    = p + total < p_end;
    const pair_desc d2 = record(p + 2u * total);
    u32x2 lead1        = lead0;
    u32x2 next1        = next0;
    uint32_t thr1      = 0u;
    float dv1          = 0.0f;
    far_part far1      = far0;
    book_part cb1      = cb0;
    if (has1) {
      lead1 = lead_codes(d1, 0u);
      next1 = lead_codes(d1, 1u);
      thr1  = a.query_kth[d1.q];
      dv1  = fetch_diff(d1);
      far1 = fetch_far(d1);
      cb1  = fetch_book(d1);
    }

    // every row of the list at least this far from the query, whatever its codes?
    bool too_far = false;
    if (by_length) {
      float part = dv0 * dv0;
#pragma unroll
      for (uint32_t x = 0; x < kFarDims; x++) { part = fmaf(far0.v[x], far0.v[x], part); }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) { part += __shfl_xor(part, off, 64); }
      const uint32_t thr_now = uint32_t(__builtin_amdgcn_readfirstlane(thr0));
      const float bound      = __uint_as_float(thr_now >= 0x80000000u ? (thr_now & 0x7fffffffu) : 0u);
      const float gap        = sqrtf(__int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(part)))) -
                        __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(far0.radius)));
      // (an unset bound reads as a NaN here: the comparison fails and the pair is screened)
      too_far = gap > 0.0f && fminf(gap * gap * a.prune_keep - a.prune_slack, a.prune_cap) > bound;
      n_far += too_far ? 1u : 0u;
    }

    if (!too_far) {
      if constexpr (PER_CLUSTER) {
        // the pair's codebook into the wave's area (the wave's own LDS accesses are performed in order)
#pragma unroll
        for (uint32_t c = 0; c < NCB; c++) { my_book[c * 64u + lane] = cb0.v[c]; }
      }
      // terms of the first four subspaces, broadcast to scalar registers once per pair; those of
      // subspaces 4..7 are read where the few tiles that get that far need them
      constexpr uint32_t NEAGER = 4 * PQ_LEN;
      float diff[NEAGER];
#pragma unroll
      for (uint32_t t = 0; t < NEAGER; t++) {
        diff[t] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(dv0), int(t)));
      }
      const uint32_t thr       = uint32_t(__builtin_amdgcn_readfirstlane(thr0));
      const uint32_t n_rows    = d0.n_rows;
      const uint32_t n_tiles   = (n_rows + 63u) >> 6;
      const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
      bool in_play             = false;
      const uint32_t full_tiles         = n_rows >> 6;
      const unsigned long long tail_rows = (1ull << (n_rows & 63u)) - 1ull;
      // A list of kMiniTiles tiles or more gets the table of its first FIRST subspaces after all
      // (the subspaces every tile looks at): 4 * FIRST entries a lane, computed as below, against
      // FIRST entries a lane and tile.  The wave reads what it wrote itself: LDS serves a wave's
      // requests in order, no barrier.
      // (Nibble codes: 16 entries a subspace, one entry a lane for the first four: always.)
      const bool tabled = BITS == 4 || n_tiles >= kMiniTiles;
      if (tabled) {
#pragma unroll
        for (uint32_t e = 0; e < uint32_t(FIRST) * BOOK / 64u; e++) {
          const vec_t b = PER_CLUSTER ? my_book[(e & 3u) * 64u + lane] : book[e * 64u + lane];
          float score   = 0.0f;
#pragma unroll
          for (int t = 0; t < PQ_LEN; t++) {
            float df;
            if constexpr (BITS == 8) {
              df = diff[(e >> 2) * PQ_LEN + t];  // 256 entries: four rounds a subspace
            } else {
              // the lane's entry belongs to subspace lane / 16, whose terms sit in lanes of `dv0`
              df = __shfl(dv0, int((lane >> 4) * uint32_t(PQ_LEN) + uint32_t(t)), 64);
            }
            df -= b[t];
            score = fmaf(df, df, score);
          }
          mini[e * 64u + lane] = traits::encode(score);
        }
      }
      // sums the leading codes `cur` of the rows of tile `tile`
      auto sum_tile = [&](auto use_table, const u32x2& cur, uint32_t tile) __attribute__((always_inline)) {
        // lanes past the list's end count only in its last, partial tile
        const unsigned long long rows = tile < full_tiles ? ~0ull : tail_rows;
        const uint32_t w[2]           = {cur.x, cur.y};
        acc_t acc        = acc_t(0);
        auto add_codes = [&](int first, int last) __attribute__((always_inline)) {
#pragma unroll
          for (int kk = first; kk < last; kk++) {
            const uint32_t c = BITS == 8 ? (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu : (w[kk >> 3] >> ((kk & 7) * 4)) & 0xfu;
            lut_t v;
            if (decltype(use_table)::value && kk < FIRST) {
              v = mini[kk * int(BOOK) + c];
            } else {
              const vec_t b = PER_CLUSTER ? my_book[c] : book[kk * int(BOOK) + c];
              float score   = 0.0f;
#pragma unroll
              for (int t = 0; t < PQ_LEN; t++) {
                float df;
                if (kk < 4) {
                  df = diff[(kk & 3) * PQ_LEN + t];
                } else {
                  int held = __float_as_int(dv0);
                  asm volatile("" : "+v"(held));  // keeps the broadcast inside the rare branch
                  df = __int_as_float(__builtin_amdgcn_readlane(held, kk * PQ_LEN + t));
                }
                df -= b[t];
                score = fmaf(df, df, score);
              }
              v = traits::encode(score);
            }
            if (OUT_HALF) {
              acc = acc_t(acc + traits::to_half(v));
            } else if (LUT == LUT_F16) {
              acc = acc_t(fmaf(traits::to_float(v), one, float(acc)));
            } else {
              acc = acc_t(acc + traits::to_float(v));
            }
          }
        };
        auto any_in_play = [&]() __attribute__((always_inline)) {
          return (__builtin_amdgcn_ballot_w64(!(__float_as_uint(float(acc)) > stop_bits)) & rows) != 0ull;
        };
        add_codes(0, FIRST);
        in_play = any_in_play();
        if (FIRST < MID && in_play) {
          add_codes(FIRST, MID);
          in_play = any_in_play();
        }
        if (in_play) {
          add_codes(MID, int(SUB));
          in_play = any_in_play();
        }
      };
      // Three registers take turns: while tile t is summed, the codes of tiles t + 1 and t + 2
      // are in flight; a register is reloaded right after the step that consumed it, and the loop
      // is unrolled by three so that none is copied while its load is outstanding.  Loads are
      // unconditional (they may run up to three tiles past the list, into the plane's slack or the
      // next lists), so the waits in the loop count outstanding loads instead of draining them.
      auto walk = [&](auto use_table) __attribute__((always_inline)) {
        u32x2 r0 = lead0, r1 = next0, r2;
        for (uint32_t tile = 0; tile < n_tiles; tile += 3u) {
          r2 = lead_codes(d0, tile + 2u);
          sum_tile(use_table, r0, tile);
          if (in_play || tile + 1u >= n_tiles) { break; }
          r0 = lead_codes(d0, tile + 3u);
          sum_tile(use_table, r1, tile + 1u);
          if (in_play || tile + 2u >= n_tiles) { break; }
          r1 = lead_codes(d0, tile + 4u);
          sum_tile(use_table, r2, tile + 2u);
          if (in_play) { break; }
        }
      };
      if (tabled) {
        walk(std::true_type{});
      } else {
        walk(std::false_type{});
      }
      if (in_play) { push_survivor(pending, n_pending, lane, d0, survivors, n_survivors, alive); }
    }

    if (!has1) { break; }
    p += total;
    d0    = d1;
    d1    = uniform(d2);
    lead0 = lead1;
    next0 = next1;
    thr0  = thr1;
    dv0   = dv1;
    far0  = far1;
    cb0   = cb1;
  }
  if (n_pending != 0) { flush_survivors(pending, n_pending, lane, survivors, n_survivors); }
  if (n_far != 0 && lane == 0) { atomicAdd(n_survivors + kFarPairsWord, n_far); }
}

template <int PQ_LEN, int LUT, bool OUT_HALF, int FIRST, int BITS, bool PER_CLUSTER = false>
void launch_screen_direct_first(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                                pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive,
                                hipStream_t stream)
{
  auto kernel       = scan_screen_direct_kernel<PQ_LEN, LUT, OUT_HALF, FIRST, BITS, PER_CLUSTER>;
  // codebooks of the leading subspaces (8 x 256 or 16 x 16 entries), a batch of survivors per wave,
  // and (byte codes) a wave's table of the first subspaces
  const size_t smem = kScreenLdsBase + size_t(kDirectSubs) * (BITS == 8 ? 256 : 32) * sizeof(typename book_vec<PQ_LEN>::type) +
                      size_t(kDirectThreads / 64u) * kSurvivorBatchBytes +
                      size_t(kDirectThreads / 64u) * FIRST * 256 * sizeof(typename lut_traits<LUT>::storage);
  // persistent blocks: exactly as many as are resident at once (per instance)
  static const int per_cu = prepare_persistent_kernel(kernel, kDirectThreads, smem, smem);
  const int n_cu          = device_cu_count();
  constexpr uint32_t wpb = kDirectThreads / 64u;
  uint32_t grid          = uint32_t(n_cu) * uint32_t(per_cu);
  const uint32_t needed  = (n_pairs + wpb - 1u) / wpb;
  if (grid > needed) { grid = needed; }
  const uint32_t n_chunks    = (a.pq_dim + 15u) / 16u;
  const uint32_t group_bytes = n_chunks * 512u;
  kernel<<<grid, kDirectThreads, smem, stream>>>(a, desc, n_pairs, group_bytes, survivors, n_survivors, alive);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER = false>
void launch_screen_direct(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                          pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive, hipStream_t stream)
{
  if constexpr (PER_CLUSTER) {
    launch_screen_direct_first<PQ_LEN, LUT, OUT_HALF, kScreenFirstCheck, 8, true>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
    return;
  }
  if constexpr (PQ_LEN == 1 || PQ_LEN == 2 || PQ_LEN == 4) {
    if (a.pq_bits == 4) {
      launch_screen_direct_first<PQ_LEN, LUT, OUT_HALF, 4, 4>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
      return;
    }
  }
  launch_screen_direct_first<PQ_LEN, LUT, OUT_HALF, kScreenFirstCheck, 8>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
}

template <int SUBS, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER>
void launch_screen_sub(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                            pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive,
                            hipStream_t stream)
{
  using lut_t       = typename lut_traits<LUT>::storage;
  auto kernel       = scan_screen_kernel<SUBS, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER>;
  const size_t smem = kScreenLdsBase + size_t(kScreenG) * SUBS * 256 * sizeof(lut_t) +
                      size_t(kScreenG) * SUBS * PQ_LEN * 4 + size_t(kScreenG) * kSurvivorBatchBytes;
  // persistent blocks: exactly as many as are resident at once (per instance)
  static const int per_cu = prepare_persistent_kernel(kernel, kScreenThreads, smem, smem);
  const int n_cu          = device_cu_count();
  const uint32_t n_iters = (n_pairs + kScreenG - 1) / kScreenG;
  uint32_t grid          = uint32_t(n_cu) * uint32_t(per_cu);
  if (grid > n_iters) { grid = n_iters; }
  const uint32_t n_chunks    = (a.pq_dim + 15u) / 16u;
  const uint32_t group_bytes = n_chunks * 512u;
  kernel<<<grid, kScreenThreads, smem, stream>>>(a, desc, n_pairs, group_bytes, survivors, n_survivors,
                                                 alive);
  CUVS_HIP_TRY(hipGetLastError());
}

constexpr uint32_t kPerClusterDirectRows = 1536;
template <int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER>
void launch_screen_instance(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                            pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive,
                            hipStream_t stream)
{
  // Per-cluster codebooks take the table-free kernel too (a wave then holds its pair's codebook),
  // but only on lists of moderate length.  What decides is how many rows get past the first
  // subspaces, each of which costs eight vector instructions here against a lookup there: lists
  // of 610 / 1,220 / 1,830 rows of the 128-dimensional benchmark rows take 0.44 / 0.71 / 0.95 ms here
  // and 0.87 / 1.27 ms with a table per pair, but lists of 2,000 rows of which a tenth survives
  // (100 M rows, 200 probes) 14.8 ms here and 11.0 ms with tables.
  if (a.lead_plane != nullptr && (!PER_CLUSTER || (a.pq_bits == 8 && a.mean_list_rows < kPerClusterDirectRows))) {
    launch_screen_direct<PQ_LEN, LUT, OUT_HALF, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
    return;
  }
  launch_screen_sub<kScreenSubs, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
}

template <int PQ_LEN, bool PER_CLUSTER>
void launch_screen_types(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                         pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive, hipStream_t s)
{
  if (!a.out_half) {
    if (a.lut_dtype == CUDA_R_32F) {
      launch_screen_instance<PQ_LEN, LUT_F32, false, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, s);
    } else if (a.lut_dtype == CUDA_R_16F) {
      launch_screen_instance<PQ_LEN, LUT_F16, false, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, s);
    } else {
      launch_screen_instance<PQ_LEN, LUT_FP8U, false, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, s);
    }
  } else {
    if (a.lut_dtype == CUDA_R_16F) {
      launch_screen_instance<PQ_LEN, LUT_F16, true, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, s);
    } else {
      launch_screen_instance<PQ_LEN, LUT_FP8U, true, PER_CLUSTER>(a, desc, n_pairs, survivors, n_survivors, alive, s);
    }
  }
}


/* ---------------------------------------------------------------------------------------------
 * Screening for inner-product and cosine searches (per-subspace codebooks, the plane of leading
 * codes; 8- and 4-bit codes).
 *
 * Table entries of these metrics have either sign, so a partial sum bounds nothing by itself.  What
 * does: entry (j, code) is LutT(x) with x = -(sum_t c_t q_t) - (sum_t q_t b_t[code]) over the
 * subspace's dimensions, whose second term depends on the query and the code alone.  With
 * U_j(q) = max over codes of that term (ip_query_bounds_kernel, once per query) every entry of
 * subspace j of a pair is at least m_j = LutT(-(sum_t c_t q_t) - U_j - rounding slack), because the
 * table's rounding is monotone.  A row whose sum over the first S subspaces is p then ends at or
 * above p + sum_{j >= S} m_j - (rounding of the remaining additions), and a pair none of whose rows
 * can still reach the query's k-th best score is dropped, exactly as under L2.  Rows are only ever
 * dropped on a proven bound, so the results are those of the full scan.
 *
 * fp32 sums: the rounding of the M additions is bounded analytically (a few 2^-24 of the sum of the
 * entries' magnitudes).  binary16 sums: the error bound of hundreds of half-precision additions
 * would be useless, but rounded addition is monotone in both operands, so the sum of a
 * hypothetical row that takes the minimum m_j in every remaining subspace, added in the scan's own
 * order and type, is a lower bound of every real row that starts from at least the same partial
 * sum.  The wave evaluates that chain for 64 starting values at once (a lane each) and takes the
 * smallest one that ends above the bound as the threshold for the rows' partial sums.
 * --------------------------------------------------------------------------------------------- */

/** out[q][j] = (U, W): the largest sum_t q_t b_t[code] over the codes of subspace j, and the largest
 *  sum_t |q_t b_t[code]| (what bounds the rounding of an entry's evaluation).  A lane per query,
 *  a block per 256 queries and kBoundSubs subspaces, whose codebooks it stages in LDS: every lane
 *  reads the same four codes at a time (a broadcast), the maxima need no exchange between lanes. */
constexpr uint32_t kBoundSubs = 4;
template <int PQ_LEN>
__global__ __launch_bounds__(256) void ip_query_bounds_kernel(const float* __restrict__ rot_q,
                                                              const float* __restrict__ pq_centers, uint32_t n_queries,
                                                              uint32_t pq_dim, uint32_t book, uint32_t rot_dim,
                                                              float2* __restrict__ out)
{
  __shared__ __align__(16) float s_book[kBoundSubs * PQ_LEN * 256];  // [subspace][component][code]
  const uint32_t q  = blockIdx.x * 256u + threadIdx.x;
  const uint32_t qr = q < n_queries ? q : n_queries - 1u;
  const float* qrow = rot_q + uint64_t(qr) * rot_dim;
  const uint32_t j0 = blockIdx.y * kBoundSubs;
  const uint32_t nj = pq_dim - j0 < kBoundSubs ? pq_dim - j0 : kBoundSubs;
  // the block's codebooks are one contiguous run of nj * PQ_LEN * book floats
  for (uint32_t x = threadIdx.x; x < nj * PQ_LEN * book; x += 256u) {
    s_book[x] = pq_centers[uint64_t(j0) * PQ_LEN * book + x];
  }
  __syncthreads();
  for (uint32_t u = 0; u < nj; u++) {
    const uint32_t j = j0 + u;
    float qv[PQ_LEN];
#pragma unroll
    for (int t = 0; t < PQ_LEN; t++) { qv[t] = qrow[j * PQ_LEN + t]; }
    const float* bj = s_book + u * PQ_LEN * book;
    float best = -FLT_MAX, mag = 0.0f;
#pragma unroll 4
    for (uint32_t code = 0; code < book; code += 4) {  // a codebook has 16 entries or more
      float dot[4] = {0.0f, 0.0f, 0.0f, 0.0f}, m[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        const float4 bv4 = *reinterpret_cast<const float4*>(bj + uint32_t(t) * book + code);
        const float bv[4] = {bv4.x, bv4.y, bv4.z, bv4.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          dot[e] = fmaf(qv[t], bv[e], dot[e]);
          m[e]   = fmaf(fabsf(qv[t]), fabsf(bv[e]), m[e]);
        }
      }
      best = fmaxf(fmaxf(best, fmaxf(dot[0], dot[1])), fmaxf(dot[2], dot[3]));
      mag  = fmaxf(fmaxf(mag, fmaxf(m[0], m[1])), fmaxf(m[2], m[3]));
    }
    if (q < n_queries) { out[uint64_t(q) * pq_dim + j] = make_float2(best, mag); }
  }
}

__device__ __forceinline__ float wave_sum_f32(float v)
{
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) { v += __shfl_xor(v, m, 64); }
  return v;
}

/** The product as its own rounded fp32 number (the table's term c q is rounded before it is
 *  subtracted: the compiler must not fuse it into the subtraction). */
__device__ __forceinline__ float rounded_product(float x, float y)
{
  float p = x * y;
  asm volatile("" : "+v"(p));
  return p;
}

template <int PQ_LEN, int LUT, bool OUT_HALF, int BITS>
__global__ __launch_bounds__(kDirectThreads, 2) void scan_screen_ip_kernel(
  scan_args a, const pair_desc* __restrict__ desc, uint32_t n_pairs, const float2* __restrict__ qbounds,
  pair_desc* __restrict__ survivors, uint32_t* __restrict__ n_survivors, uint8_t* __restrict__ alive)
{
  using traits = lut_traits<LUT>;
  using lut_t  = typename traits::storage;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  using vec_t  = typename book_vec<PQ_LEN>::type;
  static_assert(BITS == 8 || BITS == 4, "byte or nibble codes");
  constexpr uint32_t SUB  = BITS == 8 ? kDirectSubs : 2u * kDirectSubs;  // subspaces in a row's 8 leading bytes
  constexpr uint32_t BOOK = 1u << BITS;
  constexpr int FIRST     = BITS == 8 ? 2 : 4;
  constexpr int MID       = BITS == 8 ? 4 : 8;
  static_assert(SUB * PQ_LEN <= 64, "the leading subspaces' terms sit in the lanes of a register per component");
  auto* book      = reinterpret_cast<LDS_AS vec_t*>(uintptr_t(kScreenLdsBase));
  const float one = opaque_one_s();
  constexpr uint32_t off_pending = kScreenLdsBase + SUB * BOOK * uint32_t(sizeof(vec_t));
  // binary16 sums: the least entries of a pair, a binary16 number a subspace, for the wave's chain
  constexpr uint32_t off_lows = (off_pending + (kDirectThreads / 64u) * kSurvivorBatchBytes + 15u) & ~15u;

  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr uint32_t WPB = kDirectThreads / 64u;
  if (a.screen_pairs_dev != nullptr) { n_pairs = uint32_t(__builtin_amdgcn_readfirstlane(*a.screen_pairs_dev)); }
  const wave_pairs mine  = screen_wave_pairs(n_pairs, wid, WPB);
  if (mine.first - wid >= mine.end) { return; }  // the whole block, before its barrier
  for (uint32_t e = tid; e < SUB * BOOK; e += kDirectThreads) {
    vec_t v = {};
#pragma unroll
    for (int t = 0; t < PQ_LEN; t++) { v[t] = a.pq_centers[((e / BOOK) * PQ_LEN + t) * BOOK + (e % BOOK)]; }
    book[e] = v;
  }
  lds_barrier_s();
  auto* pending      = reinterpret_cast<LDS_AS uint32_t*>(uintptr_t(off_pending + wid * kSurvivorBatchBytes));
  auto* my_lows      = reinterpret_cast<LDS_AS uint16_t*>(uintptr_t(off_lows + wid * (kIpRounds * 64u * 2u)));
  uint32_t n_pending = 0;
  const auto* plane  = reinterpret_cast<const GLOBAL_AS u32x2*>(reinterpret_cast<uintptr_t>(a.lead_plane));
  const bool cosine  = a.metric == int(DistanceType::CosineExpanded);
  const uint32_t M   = a.pq_dim;

  /** The entry as the scan adds it, widened to the type of the sums. */
  auto widen = [&](float x) -> float {
    const lut_t e = traits::encode(x);
    return OUT_HALF ? float(traits::to_half(e)) : traits::to_float(e);
  };

  for (uint32_t p = mine.first; p < mine.end; p += mine.stride) {
    pair_desc d = desc[p];
    {
      const uint64_t ptr = reinterpret_cast<uint64_t>(d.data);
      const uint32_t hi  = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(ptr >> 32)));
      const uint32_t lo  = uint32_t(__builtin_amdgcn_readfirstlane(uint32_t(ptr)));
      d.data       = reinterpret_cast<const uint8_t*>((uint64_t(hi) << 32) | uint64_t(lo));
      d.q          = uint32_t(__builtin_amdgcn_readfirstlane(d.q));
      d.slot       = uint32_t(__builtin_amdgcn_readfirstlane(d.slot));
      d.label      = uint32_t(__builtin_amdgcn_readfirstlane(d.label));
      d.sample_off = uint32_t(__builtin_amdgcn_readfirstlane(d.sample_off));
      d.n_rows     = uint32_t(__builtin_amdgcn_readfirstlane(d.n_rows));
      d.row_off    = uint32_t(__builtin_amdgcn_readfirstlane(d.row_off));
    }
    const uint32_t n_rows = d.n_rows;
    if (n_rows == 0) { continue; }
    const uint32_t thr = uint32_t(__builtin_amdgcn_readfirstlane(a.query_kth[d.q]));
    // no bound yet (fewer than k candidates so far): nothing can be dropped
    const bool bounded = thr < 0xFF800000u;
    const float thr_f  = bounded ? unorder_f32(thr) : __uint_as_float(0x7F800000u);

    /* ---- the least each subspace can add: lane l takes subspaces l, l + 64, ... ---- */
    const float* qrow  = a.rot_q + uint64_t(d.q) * a.rot_dim;
    const float* crow  = a.centers_rot + uint64_t(d.label) * a.rot_dim;
    const float2* brow = qbounds + uint64_t(d.q) * M;
    float q0[PQ_LEN], tc0[PQ_LEN];  // terms of subspace `lane` (the leading subspaces are lanes 0 .. SUB - 1)
    float lows[kIpRounds];          // least entry of subspace r * 64 + lane (0 past the last subspace)
    float low_sum = 0.0f, mag_sum = 0.0f;
#pragma unroll
    for (uint32_t r = 0; r < kIpRounds; r++) {
      lows[r] = 0.0f;
      if (r * 64u >= M) { continue; }  // uniform
      const uint32_t j = r * 64u + lane;
      float low = 0.0f, mag = 0.0f;
      float qv[PQ_LEN], tcv[PQ_LEN];
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        qv[t]  = 0.0f;
        tcv[t] = 0.0f;
      }
      if (j < M) {
        float t_sum = 0.0f, t_abs = 0.0f;
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          qv[t]  = qrow[j * PQ_LEN + t];
          tcv[t] = rounded_product(crow[j * PQ_LEN + t], qv[t]);
          t_sum += tcv[t];
          t_abs += fabsf(tcv[t]);
        }
        const float2 uw = brow[j];
        mag             = t_abs + uw.y;
        // below every entry's fp32 value: the exact minimum less 2^-20 of the magnitudes (the
        // evaluation of an entry makes 2 pq_len roundings of at most 2^-24 of them each)
        const float x = -t_sum - uw.x - mag * 0x1.0p-20f;
        low           = widen(x);
        // the table's rounding may enlarge a magnitude (8-bit entries by up to an eighth)
        mag = fmaxf(mag, fabsf(low)) * 1.25f;
      }
      if (r == 0) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          q0[t]  = qv[t];
          tc0[t] = tcv[t];
        }
      }
      lows[r] = low;
      low_sum += low;
      mag_sum += mag;
    }

    /* ---- thresholds of the rows' partial sums after FIRST, MID and SUB subspaces: a row whose sum
     * is above stop[c] (binary16 sums: at or above it) after at[c] subspaces is out ---- */
    float stop[3]   = {__uint_as_float(0x7F800000u), __uint_as_float(0x7F800000u), __uint_as_float(0x7F800000u)};
    const int at[3] = {FIRST, MID, int(SUB)};
    if (bounded) {
      const float all = wave_sum_f32(low_sum);
      float rest[3];  // what the subspaces from at[c] on add at least
#pragma unroll
      for (int c = 0; c < 3; c++) {
        rest[c] = all - wave_sum_f32(lane < uint32_t(at[c]) ? lows[0] : 0.0f) + (cosine ? 1.0f : 0.0f);
      }
      if constexpr (!OUT_HALF) {
        // rounding of the scan's additions, of the sums above and of the expression below
        const float slack = float(M + 2u) * 0x1.0p-22f * (wave_sum_f32(mag_sum) + 1.0f);
#pragma unroll
        for (int c = 0; c < 3; c++) {
          stop[c] = thr_f - rest[c] + slack + (fabsf(thr_f) + fabsf(rest[c]) + 1.0f) * 0x1.0p-21f;
        }
      } else {
        // binary16 sums.  The chain of a hypothetical row that adds the least entry of every
        // subspace from at[c] on, in the scan's order and type: 21 lanes per checkpoint start it
        // from values around thr - rest[c], four units in the last place apart; the smallest start
        // that ends above the bound is the checkpoint's threshold.
        const uint32_t grp = lane >= 42u ? 2u : (lane >= 21u ? 1u : 0u);
        const float mid    = thr_f - (grp == 0 ? rest[0] : (grp == 1 ? rest[1] : rest[2]));
        int expo           = 0;
        (void)frexpf(mid, &expo);  // |mid| in [2^(expo-1), 2^expo)
        expo               = expo < -13 ? -13 : expo;
        const float step   = ldexpf(1.0f, expo - 11 + 2);  // four ulps of binary16 at mid's magnitude
        _Float16 x         = _Float16(mid + (float(lane - grp * 21u) - 13.0f) * step);
        const _Float16 start = x;
        const uint32_t from  = grp == 0 ? uint32_t(FIRST) : (grp == 1 ? uint32_t(MID) : SUB);  // the lane's first subspace
        // The terms go through the wave's LDS area (subspace j at halfword j) and come back eight
        // at a time, the same eight to every lane: an LDS read per eight additions where a
        // cross-lane read per addition doubled the chain's vector instructions.  (The wave's own
        // LDS accesses are performed in order.)
#pragma unroll
        for (uint32_t r = 0; r < kIpRounds; r++) {
          if (r * 64u >= M) { continue; }  // uniform
          my_lows[r * 64u + lane] = __builtin_bit_cast(uint16_t, _Float16(lows[r]));  // exact: a binary16 number
        }
        {
          // the leading subspaces: a lane's chain starts at its checkpoint
          const u32x4 w8a = *reinterpret_cast<const LDS_AS u32x4*>(my_lows);
          const u32x4 w8b = *reinterpret_cast<const LDS_AS u32x4*>(my_lows + 8);
          const uint32_t wd[8] = {w8a.x, w8a.y, w8a.z, w8a.w, w8b.x, w8b.y, w8b.z, w8b.w};
#pragma unroll
          for (int l = FIRST; l < int(SUB); l++) {
            const _Float16 add = __builtin_bit_cast(_Float16, uint16_t(wd[l >> 1] >> ((l & 1) * 16)));
            x = _Float16(x + (uint32_t(l) >= from ? add : _Float16(0)));
          }
        }
        // (the terms past the last subspace are zero; with four waves a SIMD the wait for a read
        // is covered: requesting sixteen terms ahead of the additions measured the same)
        for (uint32_t j = SUB; j < M; j += 8u) {
          const u32x4 w8 = *reinterpret_cast<const LDS_AS u32x4*>(my_lows + j);
          const uint32_t wd[4] = {w8.x, w8.y, w8.z, w8.w};
#pragma unroll
          for (int l = 0; l < 8; l++) {
            const _Float16 add = __builtin_bit_cast(_Float16, uint16_t(wd[l >> 1] >> ((l & 1) * 16)));
            x = _Float16(x + add);
          }
        }
        if (cosine) { x = _Float16(x + _Float16(1)); }
        // a chain is monotone in its starting value: the lanes of a group that end above the bound are an upper range
        const unsigned long long over = __builtin_amdgcn_ballot_w64(float(x) > thr_f);
        const uint32_t startbits      = uint32_t(__builtin_bit_cast(uint16_t, start));
#pragma unroll
        for (int c = 0; c < 3; c++) {
          const unsigned long long mine = over & (c == 0 ? 0x1FFFFFull : (c == 1 ? 0x1FFFFFull << 21 : ~0ull << 42));
          if (mine != 0ull) {
            stop[c] = float(__builtin_bit_cast(_Float16, uint16_t(__builtin_amdgcn_readlane(int(startbits), __builtin_ctzll(mine)))));
          }
        }
      }
    }

    /* ---- nibble codes: the entries of the first four subspaces, which every tile sums, one a lane
     * (subspace lane / 16, code lane % 16), in the form the sums take them ---- */
    float first_entry = 0.0f;
    if constexpr (BITS == 4) {
      const int kk   = int(lane >> 4);
      const vec_t b  = book[lane];  // kk * 16 + code
      float score    = 0.0f;
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        const float tc = __shfl(tc0[t], kk, 64);
        const float qv = __shfl(q0[t], kk, 64);
        score -= tc;
        score = fmaf(-qv, b[t], score);
      }
      first_entry = widen(score);
    }

    /* ---- the rows' leading codes ---- */
    const uint32_t n_tiles = (n_rows + 63u) >> 6;
    bool in_play           = false;
    u32x2 cur              = plane[uint64_t(d.row_off) + lane];
    for (uint32_t tile = 0; tile < n_tiles && !in_play; tile++) {
      // (the plane carries slack past the last list: the load needs no condition)
      const u32x2 ahead = plane[uint64_t(d.row_off) + (tile + 1u) * 64u + lane];
      const unsigned long long rows =
        tile * 64u + 64u <= n_rows ? ~0ull : (1ull << (n_rows & 63u)) - 1ull;
      const uint32_t w[2] = {cur.x, cur.y};
      acc_t acc           = acc_t(0);
      auto add_codes = [&](int first, int last) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = first; kk < last; kk++) {
          const uint32_t c = BITS == 8 ? (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu : (w[kk >> 3] >> ((kk & 7) * 4)) & 0xfu;
          const vec_t b    = book[kk * int(BOOK) + c];
          float score      = 0.0f;
#pragma unroll
          for (int t = 0; t < PQ_LEN; t++) {
            const float tc = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(tc0[t]), kk));
            const float qv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(q0[t]), kk));
            score -= tc;
            score = fmaf(-qv, b[t], score);
          }
          const lut_t v = traits::encode(score);
          if (OUT_HALF) {
            acc = acc_t(acc + traits::to_half(v));
          } else if (LUT == LUT_F16) {
            acc = acc_t(fmaf(traits::to_float(v), one, float(acc)));
          } else {
            acc = acc_t(acc + traits::to_float(v));
          }
        }
      };
      // still open: at or below the threshold (binary16 sums: below it)
      auto open = [&](int c) __attribute__((always_inline)) {
        const bool mine = OUT_HALF ? float(acc) < stop[c] : float(acc) <= stop[c];
        return (__builtin_amdgcn_ballot_w64(mine) & rows) != 0ull;
      };
      if constexpr (BITS == 4) {
        // a lane exchange per code in place of a codebook gather and the entry's arithmetic
        static_assert(BITS != 4 || FIRST == 4, "64 entries: four subspaces of sixteen codes");
#pragma unroll
        for (int kk = 0; kk < FIRST; kk++) {
          const uint32_t c  = (w[0] >> (kk * 4)) & 0xfu;
          const float entry = __int_as_float(__builtin_amdgcn_ds_bpermute(int((uint32_t(kk) * 16u + c) << 2), __float_as_int(first_entry)));
          acc               = acc_t(acc + acc_t(entry));
        }
      } else {
        add_codes(0, FIRST);
      }
      in_play = open(0);
      if (in_play) {
        add_codes(FIRST, MID);
        in_play = open(1);
      }
      if (in_play) {
        add_codes(MID, int(SUB));
        in_play = open(2);
      }
      cur = ahead;
    }
    if (in_play) { push_survivor(pending, n_pending, lane, d, survivors, n_survivors, alive); }
  }
  if (n_pending != 0) { flush_survivors(pending, n_pending, lane, survivors, n_survivors); }
}

template <int PQ_LEN, int LUT, bool OUT_HALF, int BITS>
void launch_screen_ip_instance(const scan_args& a, const pair_desc* desc, uint32_t n_pairs, const float2* qbounds,
                               pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive, hipStream_t stream)
{
  auto kernel       = scan_screen_ip_kernel<PQ_LEN, LUT, OUT_HALF, BITS>;
  const size_t smem = kScreenLdsBase + size_t(kDirectSubs) * (BITS == 8 ? 256 : 32) * sizeof(typename book_vec<PQ_LEN>::type) +
                      size_t(kDirectThreads / 64u) * kSurvivorBatchBytes + 16 +
                      size_t(kDirectThreads / 64u) * kIpRounds * 64u * 2u;
  static const int per_cu = prepare_persistent_kernel(kernel, kDirectThreads, smem, smem);
  constexpr uint32_t wpb = kDirectThreads / 64u;
  uint32_t grid          = uint32_t(device_cu_count()) * uint32_t(per_cu);
  const uint32_t needed  = (n_pairs + wpb - 1u) / wpb;
  if (grid > needed) { grid = needed; }
  kernel<<<grid, kDirectThreads, smem, stream>>>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int PQ_LEN, int BITS>
void launch_screen_ip_types(const scan_args& a, const pair_desc* desc, uint32_t n_pairs, const float2* qbounds,
                            pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive, hipStream_t s)
{
  if (!a.out_half) {
    if (a.lut_dtype == CUDA_R_32F) {
      launch_screen_ip_instance<PQ_LEN, LUT_F32, false, BITS>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, s);
    } else if (a.lut_dtype == CUDA_R_16F) {
      launch_screen_ip_instance<PQ_LEN, LUT_F16, false, BITS>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, s);
    } else {
      launch_screen_ip_instance<PQ_LEN, LUT_FP8S, false, BITS>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, s);
    }
  } else {
    if (a.lut_dtype == CUDA_R_16F) {
      launch_screen_ip_instance<PQ_LEN, LUT_F16, true, BITS>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, s);
    } else {
      launch_screen_ip_instance<PQ_LEN, LUT_FP8S, true, BITS>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, s);
    }
  }
}

}  // namespace

uint32_t scan_screen_bytes_per_row(bool per_cluster, bool lead_plane)
{
  (void)per_cluster;
  (void)lead_plane;
  return kScreenSubs <= 8 ? 8u : 16u;
}

bool scan_screen_ip(const scan_args& a)
{
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (!ip || !a.fused || (a.pq_bits != 8 && a.pq_bits != 4) || a.pq_dim < 32) { return false; }
  if (a.lut_dtype == CUDA_R_32F && a.out_half) { return false; }
  // per-subspace codebooks (the bound's query part is per query then) and the plane of leading codes
  if (a.per_cluster || a.lead_plane == nullptr || a.rot_dim != a.pq_dim * a.pq_len) { return false; }
  if (a.pq_dim > 64u * kIpRounds) { return false; }
  return a.pq_len == 1 || a.pq_len == 2 || a.pq_len == 4;
}

/*
 * The surviving records class by class, as a counting sort without global atomics: every block
 * counts the classes of its contiguous run of records in LDS (order_survivors_count_kernel); every
 * block then finds where its records of each class go from the table of (block, class) counts and
 * moves them (order_survivors_move_kernel).  Records that follow each other in the input (the
 * survivors of one list, as a rule) stay neighbours.
 */
constexpr uint32_t kOrderSurvivorThreads = 256;
constexpr uint32_t kOrderSurvivorBlocks  = 64;
static_assert(kOrderSurvivorThreads == kSurvivorClasses, "a thread per class in the scans");
static_assert(kSurvivorTable + kOrderSurvivorBlocks * kSurvivorClasses <= kSurvivorWords, "table of counts");

__global__ __launch_bounds__(kOrderSurvivorThreads) void order_survivors_count_kernel(
  const pair_desc* __restrict__ survivors, uint32_t* __restrict__ words)
{
  __shared__ uint32_t hist[kSurvivorClasses];
  const uint32_t tid = threadIdx.x;
  hist[tid]          = 0;
  __syncthreads();
  const uint32_t n   = words[0];
  const uint32_t per = (n + gridDim.x - 1u) / gridDim.x;
  const uint32_t i0  = blockIdx.x * per;
  const uint32_t i1  = i0 + per < n ? i0 + per : n;
  for (uint32_t i = i0 + tid; i < i1; i += kOrderSurvivorThreads) {
    atomicAdd(&hist[class_of_rows(survivors[i].n_rows)], 1u);
  }
  __syncthreads();
  words[kSurvivorTable + blockIdx.x * kSurvivorClasses + tid] = hist[tid];
}

__global__ __launch_bounds__(kOrderSurvivorThreads) void order_survivors_move_kernel(
  const pair_desc* __restrict__ survivors, const uint32_t* __restrict__ words, pair_desc* __restrict__ ordered)
{
  __shared__ uint32_t start[kSurvivorClasses];
  __shared__ uint32_t wave_sums[kOrderSurvivorThreads / 64];
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wid = tid >> 6;
  // thread = class: records of the class in all blocks, and in the blocks before this one
  uint32_t total = 0, before = 0;
#pragma unroll 8
  for (uint32_t b = 0; b < kOrderSurvivorBlocks; b++) {
    const uint32_t c = words[kSurvivorTable + b * kSurvivorClasses + tid];
    total += c;
    before += b < blockIdx.x ? c : 0u;
  }
  const uint32_t incl = wave_inclusive_scan(total);
  if (lane == 63u) { wave_sums[wid] = incl; }
  __syncthreads();
  uint32_t classes_before = 0;
  for (uint32_t w = 0; w < wid; w++) { classes_before += wave_sums[w]; }
  start[tid] = classes_before + incl - total + before;
  __syncthreads();
  const uint32_t n   = words[0];
  const uint32_t per = (n + gridDim.x - 1u) / gridDim.x;
  const uint32_t i0  = blockIdx.x * per;
  const uint32_t i1  = i0 + per < n ? i0 + per : n;
  for (uint32_t i = i0 + tid; i < i1; i += kOrderSurvivorThreads) {
    const u32x4* src = reinterpret_cast<const u32x4*>(survivors + i);
    const u32x4 lo = src[0], hi = src[1];
    const uint32_t pos = atomicAdd(&start[class_of_rows(hi.z)], 1u);  // hi.z: n_rows
    u32x4* dst = reinterpret_cast<u32x4*>(ordered + pos);
    dst[0]     = lo;
    dst[1]     = hi;
  }
}

void launch_order_survivors(const pair_desc* survivors, uint32_t* n_survivors, pair_desc* ordered,
                            hipStream_t stream)
{
  static_assert(offsetof(pair_desc, n_rows) == 24, "n_rows is the third word of the record's second half");
  order_survivors_count_kernel<<<kOrderSurvivorBlocks, kOrderSurvivorThreads, 0, stream>>>(survivors, n_survivors);
  CUVS_HIP_TRY(hipGetLastError());
  order_survivors_move_kernel<<<kOrderSurvivorBlocks, kOrderSurvivorThreads, 0, stream>>>(survivors, n_survivors, ordered);
  CUVS_HIP_TRY(hipGetLastError());
}

bool scan_screen_supported(const scan_args& a)
{
  if (scan_screen_ip(a)) { return true; }
  const bool l2 = a.metric == int(DistanceType::L2Expanded) || a.metric == int(DistanceType::L2SqrtExpanded);
  if (!l2 || !a.fused || (a.pq_bits != 8 && a.pq_bits != 4) || a.pq_dim < 32) { return false; }
  if (a.lut_dtype == CUDA_R_32F && a.out_half) { return false; }
  if (a.pq_bits == 4) {
    // nibble codes: only the table-free kernel on the plane of leading code bytes reads them
    return !a.per_cluster && a.lead_plane != nullptr && a.lut_dtype != CUDA_R_32F &&
           (a.pq_len == 1 || a.pq_len == 2 || a.pq_len == 4);
  }
  return a.pq_len == 1 || a.pq_len == 2 || a.pq_len == 3 || a.pq_len == 4 || a.pq_len == 8;
}

size_t scan_screen_scratch_bytes(const scan_args& a, uint32_t n_queries)
{
  return scan_screen_ip(a) ? size_t(n_queries) * a.pq_dim * sizeof(float2) : 0;
}

void launch_scan_screen(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                        pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive, void* scratch,
                        hipStream_t stream)
{
  CUVS_EXPECTS(scan_screen_supported(a), "the screening pass does not cover these search arguments");
  if (n_pairs == 0) { return; }
  if (scan_screen_ip(a)) {
    CUVS_EXPECTS(scratch != nullptr, "the screen of an inner-product search needs its scratch buffer");
    auto* qbounds = static_cast<float2*>(scratch);
    {
      const dim3 grid((a.n_queries + 255u) / 256u, (a.pq_dim + kBoundSubs - 1u) / kBoundSubs);
      const uint32_t book = 1u << a.pq_bits;
      switch (a.pq_len) {
        case 1: ip_query_bounds_kernel<1><<<grid, 256, 0, stream>>>(a.rot_q, a.pq_centers, a.n_queries, a.pq_dim, book, a.rot_dim, qbounds); break;
        case 2: ip_query_bounds_kernel<2><<<grid, 256, 0, stream>>>(a.rot_q, a.pq_centers, a.n_queries, a.pq_dim, book, a.rot_dim, qbounds); break;
        default: ip_query_bounds_kernel<4><<<grid, 256, 0, stream>>>(a.rot_q, a.pq_centers, a.n_queries, a.pq_dim, book, a.rot_dim, qbounds); break;
      }
    }
    CUVS_HIP_TRY(hipGetLastError());
    auto by_bits = [&](auto len) {
      constexpr int PQ_LEN = decltype(len)::value;
      if (a.pq_bits == 8) {
        launch_screen_ip_types<PQ_LEN, 8>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, stream);
      } else {
        launch_screen_ip_types<PQ_LEN, 4>(a, desc, n_pairs, qbounds, survivors, n_survivors, alive, stream);
      }
    };
    switch (a.pq_len) {
      case 1: by_bits(std::integral_constant<int, 1>{}); break;
      case 2: by_bits(std::integral_constant<int, 2>{}); break;
      default: by_bits(std::integral_constant<int, 4>{}); break;
    }
    return;
  }
  auto by_kind = [&](auto len) {
    constexpr int PQ_LEN = decltype(len)::value;
    if (a.per_cluster) {
      launch_screen_types<PQ_LEN, true>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
    } else {
      launch_screen_types<PQ_LEN, false>(a, desc, n_pairs, survivors, n_survivors, alive, stream);
    }
  };
  switch (a.pq_len) {
    case 1: by_kind(std::integral_constant<int, 1>{}); break;
    case 2: by_kind(std::integral_constant<int, 2>{}); break;
    case 3: by_kind(std::integral_constant<int, 3>{}); break;
    case 4: by_kind(std::integral_constant<int, 4>{}); break;
    default: by_kind(std::integral_constant<int, 8>{}); break;
  }
}

}  // namespace cuvs::neighbors::ivf_pq::detail
