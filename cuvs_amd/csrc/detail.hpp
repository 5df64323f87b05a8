/*
 * Internal declarations shared by the host driver and the HIP kernels of the IVF-PQ search path.
 */
#pragma once

#include <cuvs/core/resources.hpp>
#include <cuvs/neighbors/ivf_pq.hpp>

#include <hip/hip_runtime_api.h>

#include "memory.hpp"

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>
#include <mutex>
#include <vector>

namespace cuvs {

[[noreturn]] inline void fail(const char* fmt, ...)
{
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  throw logic_error(buf);
}

#define CUVS_EXPECTS(cond, ...) \
  do {                          \
    if (!(cond)) { ::cuvs::fail(__VA_ARGS__); } \
  } while (0)

#define CUVS_HIP_TRY(call)                                                                  \
  do {                                                                                      \
    hipError_t status_ = (call);                                                            \
    if (status_ != hipSuccess) {                                                            \
      ::cuvs::fail("HIP error at %s:%d: %s (%s)", __FILE__, __LINE__, hipGetErrorName(status_), \
                   hipGetErrorString(status_));                                             \
    }                                                                                       \
  } while (0)

/** Owning device allocation out of the process's current memory source. */
struct device_buffer {
  void* ptr    = nullptr;
  size_t bytes = 0;
  device_buffer() = default;
  explicit device_buffer(size_t n) { allocate(n); }
  ~device_buffer() { release(); }
  device_buffer(const device_buffer&)            = delete;
  device_buffer& operator=(const device_buffer&) = delete;
  device_buffer(device_buffer&& o) noexcept : ptr(o.ptr), bytes(o.bytes)
  {
    o.ptr   = nullptr;
    o.bytes = 0;
  }
  device_buffer& operator=(device_buffer&& o) noexcept
  {
    if (this != &o) {
      release();
      ptr     = o.ptr;
      bytes   = o.bytes;
      o.ptr   = nullptr;
      o.bytes = 0;
    }
    return *this;
  }
  void allocate(size_t n)
  {
    release();
    if (n > 0) {
      ptr   = memory::allocate(n);
      bytes = n;
    }
  }
  void release()
  {
    memory::deallocate(ptr);
    ptr   = nullptr;
    bytes = 0;
  }
  template <typename T>
  T* as() const
  {
    return static_cast<T*>(ptr);
  }
};

inline uint32_t round_up_u32(uint32_t v, uint32_t m) { return ((v + m - 1) / m) * m; }
inline uint64_t round_up_u64(uint64_t v, uint64_t m) { return ((v + m - 1) / m) * m; }
inline uint32_t next_pow2(uint32_t v)
{
  uint32_t p = 1;
  while (p < v) { p <<= 1; }
  return p;
}

}  // namespace cuvs

namespace cuvs::neighbors::ivf_pq::detail {

using cuvs::distance::DistanceType;

/** Index contents.  Lists live in two arenas (codes, ids); list `l` starts at row `row_offset[l]`
 *  (a multiple of 32) and owns round_up(size, 32) rows. */
/** What the early-stop screen achieved on an index lately, fed back to the searches that decide
 *  whether to use it: on data whose lists all lie about as far from a query as its nearest one, the
 *  screen keeps nearly every pair and its launches only add to the scan.  One screened search at a
 *  time is observed (its survivor count is copied to pinned memory behind the search; a later
 *  search folds it in once it has landed - nothing waits), and while the verdict for the same
 *  (n_probes, k) is "does not pay", searches in the automatic mode scan plainly, except every
 *  kScreenRecheck-th one, which is screened and observed again. */
struct screen_feedback {
  static constexpr uint32_t kScreenRecheck = 64;
  static constexpr double kKeepLimit       = 0.7;  // survivors / screened pairs above which the screen is off
  std::mutex mu;
  uint32_t* host    = nullptr;  // pinned: survivors of the search under observation
  hipEvent_t landed = nullptr;  // recorded behind the copy into `host`
  bool pending      = false;
  uint64_t pending_pairs  = 0;  // pairs that search screened
  bool pending_far        = false;  // that search left far pairs out before the screen
  uint32_t pending_probes = 0, pending_k = 0;
  /** Verdicts by (n_probes, k), the most recently used first: callers that alternate between a few
   *  parameter sets each keep theirs. */
  struct verdict {
    uint32_t probes = 0, k = 0;    // 0: unused entry
    bool off                = false;
    uint32_t plain_searches = 0;   // since the verdict
    uint32_t screened_searches = 0;  // with the screen on
    // the screening kernel alone does not pay: of the pairs that the bound on their lists'
    // distance leaves over, it kept most (the early stop then runs without it)
    bool screen_off           = false;
    uint32_t unscreened_searches = 0;  // since that verdict
  };
  /** With a verdict for the screen, every kObserveEvery-th screened search is observed (the copy of
   *  the survivor count is a launch of its own on the search's stream). */
  static constexpr uint32_t kObserveEvery = 8;
  static constexpr int kVerdicts = 8;
  verdict verdicts[kVerdicts];
  /** The entry of (probes, k), moved to the front; null when there is none. */
  verdict* find(uint32_t probes, uint32_t k);
  /** The pinned word and the event (allocates; called when an index is made, never by a search). */
  void create();
  /** Folds in an observation that has landed.  Call with `mu` held. */
  void collect();
  screen_feedback() = default;
  screen_feedback(const screen_feedback&)            = delete;
  screen_feedback& operator=(const screen_feedback&) = delete;
  ~screen_feedback();
};

struct index_impl {
  index_impl();
  ~index_impl();
  index_impl(const index_impl&)            = delete;
  index_impl& operator=(const index_impl&) = delete;
  DistanceType metric        = DistanceType::L2Expanded;
  codebook_gen codebook_kind = codebook_gen::PER_SUBSPACE;
  bool conservative_memory_allocation = false;
  uint32_t n_lists = 0, dim = 0, pq_bits = 0, pq_dim = 0;
  uint32_t dim_ext = 0, pq_len = 0, rot_dim = 0, book_size = 0;
  uint32_t n_chunks = 0;  // 16-byte chunks per encoded row

  device_buffer centers, centers_rot, rotation, rotation_t, pq_centers;
  device_buffer centers_t;  // [dim_ext][coarse_pad(n_lists)]: centres k-major for the matrix-core kernel
  // two-precision probe selection: centres as binary16 [coarse_pad(n_lists)][k_pad], their stored
  // norms, and the largest centre length / |stored norm| (coarse_fast_ok: all finite and within
  // binary16's range)
  device_buffer centers_h, center_norms;
  device_buffer centers_i8;  // [coarse_i8_words(dim)][coarse_pad(n_lists)] words: centres for the 8-bit coarse search
  float c_max = 0.0f, n_max = 0.0f;
  bool coarse_fast_ok = false;
  /** centers_t, centers_h, center_norms and the maxima from `centers` (synchronises). */
  void refresh_coarse(hipStream_t stream);
  bool rotation_is_identity = false;

  device_buffer codes_arena, ids_arena;
  /** 8-bit codes (also the byte-wide copy of narrower ones) and 4-bit codes: the first eight code
   *  bytes of every row slot, packed (8 bytes per row next to the arena's n_chunks * 16): the
   *  early-stop screen decides on these alone, and reading them here touches half the cache lines
   *  the interleaved arena would, in whole lines.  Rebuilt whenever the arena changes; empty for
   *  other code widths, for 4-bit codes with conservative_memory_allocation, or with 2^32 and more
   *  row slots. */
  device_buffer lead_plane;
  /** 5 - 7 bit codes: the lists once more with a byte per code, in the layout of an 8-bit index
   *  (n_chunks8 = ceil(pq_dim / 16) chunks a row), their pointer table, and the codebooks padded to
   *  256 entries.  A search whose 256-entry table fits the byte-wide kernels then runs on these as
   *  if the index had 8-bit codes (same table entries for the codes that occur, same order of
   *  summation: same results), early stop included; the packed lists stay what every other
   *  function reads and writes.  Costs 8 / pq_bits times the packed lists' memory; not kept with
   *  conservative_memory_allocation.  Rebuilt with the lead plane. */
  device_buffer codes8_arena, data_ptrs8, pq_centers8;
  uint32_t n_chunks8 = 0;
  bool wide() const { return codes8_arena.bytes != 0; }
  std::vector<uint32_t> h_list_sizes;
  std::vector<uint64_t> h_row_offsets;  // [n_lists + 1], in rows, multiples of 32
  device_buffer list_sizes, data_ptrs, inds_ptrs;
  /** Position of every list among all lists by size, largest first (ties by list number): the
   *  order in which the search takes the pairs of each query's leading probe, long lists first. */
  device_buffer list_rank;
  /** Per list, the largest length of a row's decoded residual (rotated space), rounded up: a row
   *  of list l is at least |query - centre| - list_radius[l] away from a query, which lets an L2
   *  search drop a (query, list) pair without reading a row.  Kept with the other copies derived
   *  from the list codes (rebuild_lead_plane / refresh_derived_rows). */
  device_buffer list_radius;
  /** Per list (float4): the stored squared norm of the centre, |c_rot|^2 and |R^T c_rot - c|: with
   *  the probe selection's score they give |rotated query - rotated centre| without a pass over the
   *  dimensions (scan_far.hip).  Made with list_radius.  rotation_bounded: no row of the rotation
   *  matrix is longer than 2 (the rounding allowance of that estimate assumes it). */
  device_buffer center_terms;
  bool rotation_bounded = false;
  std::vector<int64_t> accum_sorted_sizes;  // [n_lists + 1]
  int64_t size = 0;
  mutable screen_feedback feedback;

  uint64_t group_bytes() const { return uint64_t(n_chunks) * kIndexGroupSize * kIndexGroupVecLen; }
  /** Recompute pointer tables, device sizes and the sorted prefix sums from the host vectors
   *  (role of ivf::detail::recompute_internal_state, cpp/src/neighbors/ivf_common.cuh:255-290). */
  void recompute_internal_state(hipStream_t stream);
  /** Refill `lead_plane` and the byte-wide copy of narrower codes from the codes arena (after the
   *  arena's contents changed). */
  void rebuild_lead_plane(hipStream_t stream);
  /** The same for the rows of one list that were written in place (all of it if a list has moved
   *  since the copies were made). */
  void refresh_derived_rows(uint32_t label, hipStream_t stream);
  std::vector<uint64_t> derived_offsets;  // h_row_offsets at the time the copies were made
  /** Set when list memory was written through a bare pointer (codepacker::pack on a buffer of this
   *  index): what the index derives from its lists is then refreshed by the next search, under
   *  `derived_mu`. */
  mutable std::atomic<bool> derived_stale{false};
  mutable std::mutex derived_mu;
};

/** Tells the index whose codes arena holds `list_data` (if any) that its lists were written behind
 *  its back. */
void mark_lists_written(const void* list_data);

void init_index(index_impl& ix, const index_params& params, uint32_t dim);

/* ------------------------------------------------------------------------------------------ */
/* kernel launchers (kernels.hip)                                                              */
/* ------------------------------------------------------------------------------------------ */

void launch_fill_u32(uint32_t* dst, uint32_t value, uint64_t n, hipStream_t stream);

/** qf[q, d] = mapping<float>(queries[q, d])  (detail/ann_utils.cuh:168-201) */
void launch_map_queries(const void* queries, elem_type type, uint64_t n_elems, float* out,
                        hipStream_t stream);

/** scores[q, l] = alpha * (sum_d centers[l, d] * qf[q, d] + centers[l, dim] * qnorm), fp32 FMA in
 *  ascending d.  half_inputs rounds both operands to binary16 first and the result to binary16. */
void launch_coarse_scores(const float* qf, const float* centers, uint32_t n_queries,
                          uint32_t n_lists, uint32_t dim, uint32_t dim_ext, bool ip_like,
                          bool half_inputs, float* scores, hipStream_t stream);

/** probes[q, 0..P) = lists with the P smallest (score, list id), ascending. */
/** Matrix-core variant of launch_coarse_scores (coarse.hip); same values bit for bit.  Operands are
 *  k-major with the leading dimensions padded to coarse_pad(): `qt` = [dim_ext][coarse_pad(n_queries)]
 *  from launch_map_queries_t, `ct` = [dim_ext][coarse_pad(n_lists)] from launch_transpose_centers. */
uint32_t coarse_pad(uint32_t n);
void launch_transpose_centers(const float* centers, uint32_t n_lists, uint32_t dim_ext, float* ct,
                              hipStream_t stream);
void launch_map_queries_t(const void* queries, elem_type type, uint32_t n_queries, uint32_t dim,
                          uint32_t dim_ext, bool ip_like, float* qt, hipStream_t stream);
void launch_coarse_scores_mfma(const float* qt, const float* ct, uint32_t n_queries, uint32_t n_lists,
                               uint32_t dim_ext, bool ip_like, bool half_inputs, float* scores,
                               hipStream_t stream);
/** The probe selection reads whole segments of 256 x 64 scores: the score buffer must have this
 *  many readable bytes after its last row. */
constexpr size_t kSelectSlackBytes = 256 * 64 * 4;
/** With `only` non-null, queries whose byte there is zero are left alone.  Beyond kSelectLdsProbes
 *  probes the selection's output does not fit a block's LDS: `scratch` then has
 *  select_probes_scratch_bytes(n_queries, n_probes) bytes. */
constexpr uint32_t kSelectLdsProbes = 8192;
size_t select_probes_scratch_bytes(uint32_t n_queries, uint32_t n_probes);
void launch_select_probes(const float* scores, uint32_t n_queries, uint32_t n_lists,
                          uint32_t n_probes, uint32_t* probes, hipStream_t stream,
                          const uint8_t* only = nullptr, void* scratch = nullptr);

/* coarse search in 8-bit integers (coarse_i8.hip): 32-bit words of the quantised centre rows,
 * word-major, and scores written as floats that order like the integer scores */
uint32_t coarse_i8_words(uint32_t dim);
void launch_pack_centers_i8(const float* centers, uint32_t n_lists, uint32_t dim, uint32_t dim_ext,
                            uint32_t* ct8, hipStream_t stream);
void launch_coarse_scores_i8(const float* qf, const uint32_t* ct8, uint32_t n_queries, uint32_t n_lists,
                             uint32_t dim, bool ip_like, float* scores, hipStream_t stream);

/* probe selection in two precisions (coarse_fast.hip) */
struct coarse_fast_args {
  const void* queries;     // [n_queries, dim] of `type` (f16, i8 or u8)
  elem_type type;
  uint32_t n_queries, n_lists, dim, dim_ext, n_probes;
  bool ip_like;
  const float* centers;    // [n_lists, dim_ext]
  const _Float16* ch;      // [coarse_pad(n_lists), k_pad] centres as binary16
  const float* cn;         // [coarse_pad(n_lists)] stored squared norms
  float c_max, n_max;      // largest centre length, largest |stored norm|
  float* qf;               // [n_queries, dim] out: the mapped queries in fp32 (null: not wanted)
  _Float16* qh;            // [coarse_pad(n_queries), k_pad]
  float* qnorm;            // [coarse_pad(n_queries)]
  float* minima;           // [n_queries, coarse_fast_groups(n_lists)]
  float* thr;              // [n_queries]
  uint32_t* cand_count;    // [coarse_pad(n_queries)]
  uint32_t* cand;          // [n_queries, coarse_fast_cand_cap()]
  uint8_t* fallback;       // [round_up(n_queries, 4)]
  float* scores;           // [n_queries, n_lists]: rows of flagged queries only
  uint32_t* probes;        // [n_queries, n_probes]
  float* probe_scores;     // [n_queries, n_probes] out: the probes' fp32 scores (null: not wanted; not
                           // written for the flagged queries)
};
uint32_t coarse_fast_k_pad(uint32_t dim);
uint32_t coarse_fast_max_dim();
uint32_t coarse_fast_groups(uint32_t n_lists);
uint32_t coarse_fast_cand_cap();
/** stats (3 words, device): bit patterns of the largest |element|, |stored norm| and centre length. */
void launch_pack_centers_f16(const float* centers, uint32_t n_lists, uint32_t dim, uint32_t dim_ext,
                             _Float16* ch, float* cn, uint32_t* stats, hipStream_t stream);
void launch_coarse_fast(const coarse_fast_args& a, hipStream_t stream);

/** rot_q = rotation * qf (+ row normalisation for cosine); rotation_t is [dim, rot_dim].
 *  `operand_dtype` is the coarse search's type, whose query rows and copy of the rotation matrix
 *  the reference's rotation GEMM takes (ivf_pq_search.cuh:996-1019): CUDA_R_32F as they are,
 *  CUDA_R_16F both rounded to binary16, CUDA_R_8I both as trunc(clamp(128 x)) with the integer
 *  dot product scaled by 1 / 128^2. */
void launch_rotate(const float* qf, const float* rotation_t, uint32_t n_queries, uint32_t dim,
                   uint32_t rot_dim, bool identity, bool normalize, int operand_dtype, float* rot_q,
                   hipStream_t stream);

/** chunk_indices[q, p] = inclusive prefix sum of list_sizes[probes[q, p]]; n_samples[q] = total.
 *  When `stats` is non-null (kStatSlots x 4 words), query q adds the scanned bytes, the rows and
 *  the bytes of its leading probes to words 0, 1, 2 of slot q % kStatSlots.  `query_max`
 *  (n_queries words) is filled with 0xFFFFFFFF and the `n_zero_words` words at `zero_words` with 0
 *  when given. */
constexpr uint32_t kStatSlots = 256;
void launch_chunk_indices(const uint32_t* list_sizes, const uint32_t* probes, uint32_t n_queries,
                          uint32_t n_probes, uint32_t row_chunk_bytes, uint32_t* chunk_indices,
                          uint32_t* n_samples, unsigned long long* stats, uint32_t lead_probes,
                          uint32_t* query_max, uint32_t* zero_words, uint32_t n_zero_words, hipStream_t stream);

/** Everything the scan needs to know about one (query, probe) pair, gathered once so that the
 *  scan kernel reads one 32-byte record instead of chasing four dependent pointers. */
struct pair_desc {
  const uint8_t* data;  // interleaved codes of the probed list
  uint32_t q;           // query index inside the batch
  uint32_t slot;        // q * n_probes + p: position of the pair's output
  uint32_t label;       // probed list
  uint32_t sample_off;  // sample number of the list's first row for this query
  uint32_t n_rows;      // list size
  uint32_t row_off;     // the list's first row slot in the arenas (low 32 bits)
};
static_assert(sizeof(pair_desc) == 32, "pair_desc must stay 32 bytes");

/** pair_order = ids of the (query, probe) pairs grouped by probed list; when `desc` is non-null the
 *  record of every pair is written at the same position.  With `lead_probes` < n_probes the pairs
 *  of each query's first `lead_probes` probes come first (n_queries * lead_probes records, grouped
 *  by list) and the others after them (grouped by list again); `alive`, when non-null, gets one
 *  byte per pair slot: 1 for the leading pairs, 0 for the others.  `counters` is scratch of
 *  4 * n_lists + 4 words, `sort_scratch` of order_pairs_scratch_bytes() bytes (256-byte aligned;
 *  null: the order is made with global atomics).  `list_rank` (n_lists words, a permutation; null:
 *  the identity) gives the order of the groups of leading pairs: group of list l at position
 *  list_rank[l]. */
size_t order_pairs_scratch_bytes(uint32_t n_pairs, uint32_t n_probes, uint32_t n_lists, uint32_t lead_probes);
void launch_order_pairs(const uint32_t* probes, const uint32_t* chunk_indices,
                        const uint8_t* const* data_ptrs, const int64_t* const* inds_ptrs,
                        const int64_t* ids_base, uint32_t n_pairs, uint32_t n_probes,
                        uint32_t n_lists, uint32_t* counters, void* sort_scratch, uint32_t* pair_order,
                        pair_desc* desc, uint32_t lead_probes, uint8_t* alive, bool natural_order,
                        const uint32_t* list_rank, hipStream_t stream);

struct scan_args {
  uint32_t n_queries, n_probes, k, max_samples;
  uint32_t rot_dim, pq_dim, pq_len, pq_bits;
  int metric;          // DistanceType
  int per_cluster;     // codebook kind
  int lut_dtype;       // CUDA_R_32F / 16F / 8U
  int out_half;        // internal distance dtype is fp16
  int fused;           // per-pair top-k in the kernel
  const float* rot_q;           // [n_queries, rot_dim]
  const float* centers_rot;     // [n_lists, rot_dim]
  const float* pq_centers;
  const uint8_t* const* data_ptrs;
  const int64_t* const* inds_ptrs;
  const uint32_t* list_sizes;
  const uint32_t* probes;         // [n_queries, n_probes]
  const uint32_t* chunk_indices;  // [n_queries, n_probes]
  const uint32_t* pair_order;     // [n_queries * n_probes] or null
  const pair_desc* desc;          // records of the pairs to scan, in launch order, or null
  uint32_t n_pairs;               // number of records in `desc` (persistent kernels)
  const uint32_t* n_pairs_dev;    // when non-null the number of records is read from here instead
  const uint32_t* filter_bits;    // or null
  int64_t filter_nbits;
  uint32_t* query_kth;            // [n_queries] ordered-score upper bounds (fused)
  unsigned long long* out_keys;   // fused: [n_queries, n_probes, k]
  float* out_scores;              // non-fused: [n_queries, max_samples]
  void* global_lut;               // generic kernel: table scratch when it does not fit LDS, or null
  const uint64_t* lead_plane;     // first eight code bytes of every row slot (8- and 4-bit codes), or null
  int subset;                     // generic kernel: scan the pairs of desc[0 .. n_pairs) (or *n_pairs_dev) only
  uint32_t mean_list_rows;        // rows of the index over its lists (which screening kernel pays)
  int rare_exits;                 // few tiles of this launch are expected to end early (the leading and the
                                  // surviving pairs of an early stop): the wave-per-pair kernel then has a
                                  // tile's next step on its way instead of the next tile's first one
  // The screens of an L2 search drop a pair without reading a row when every row of the list is
  // provably too far: a row's sum of entries is, in exact arithmetic, |r - b|^2 >= (|r| - |b|)^2
  // for the pair's residual r = rotated query - rotated centre and the row's decoded residual b,
  // and |b| <= list_radius[list].  prune_keep (below 1) and prune_slack cover what the table's
  // type and the sums' type can lose against exact arithmetic, prune_cap what a sum is sure to
  // reach once an entry saturates (8-bit tables): the pair goes if
  // min((|r| - radius)^2 * prune_keep - prune_slack, prune_cap) is past the query's bound.
  // prune_keep 0: not used.
  const float* list_radius;       // [n_lists], or null
  float prune_keep, prune_slack, prune_cap;
  const uint32_t* screen_pairs_dev;  // screens: when non-null the number of records is read from here
};
/** LDS bytes the scan kernel needs for these arguments (without the table when `global_lut` is
 *  set), the bytes of one lookup table, and the number of blocks (= table slices) the generic
 *  kernel runs with a global table. */
size_t scan_lds_bytes(const scan_args& a);
size_t scan_lut_bytes(const scan_args& a);
uint32_t scan_global_lut_blocks();
void launch_scan(const scan_args& a, hipStream_t stream);
/* training (train.hip) */
/** dst row i = src row i * ratio + hash(i, seed) % ratio, rows of `row_bytes` bytes. */
void launch_gather_rows(const void* src, uint64_t row_bytes, uint64_t n_out, uint64_t ratio,
                        uint32_t seed, void* dst, hipStream_t stream);
/** ext [n_lists, dim_ext] = (centre, squared norm, zeros) from flat [n_lists, dim]. */
void launch_set_centers(const float* flat, uint32_t n_lists, uint32_t dim, uint32_t dim_ext, float* ext,
                        hipStream_t stream);
void launch_accumulate(const float* x, const uint32_t* labels, uint64_t n_rows, uint32_t dim,
                       float* sums, uint32_t* counts, uint32_t* member, hipStream_t stream);
void launch_finish_centers(const float* sums, const uint32_t* counts, uint32_t n_lists, uint32_t dim,
                           bool normalize, float* flat, hipStream_t stream);
void launch_adjust_centers(const uint32_t* receivers, const uint32_t* donors, uint32_t n_pairs,
                           const float* x, const uint32_t* member, uint32_t dim, float offset,
                           float* flat, hipStream_t stream);
void launch_residuals(const float* x, const uint32_t* labels, const float* centers_ext, uint64_t n_rows,
                      uint32_t dim, uint32_t dim_ext, float* diff, hipStream_t stream);
uint32_t train_codebook_max_pq_len();
/** One balanced k-means per group (subspace or list) of `book` entries; output layout
 *  [group][pq_len][book]. */
void launch_train_codebooks(const float* res, uint32_t rot_dim, uint32_t pq_dim, uint32_t pq_len,
                            uint32_t book, bool per_cluster, uint32_t n_groups, uint32_t n_rows,
                            const uint32_t* rows, const uint32_t* offsets, uint32_t max_samples,
                            uint32_t n_iters, uint32_t seed, float* pq_centers, hipStream_t stream);

/** plane[slot] = first eight bytes of row slot `slot` of an arena of 8-bit codes. */
/** The packed codes of `n_slots` row slots as bytes in the 8-bit layout; codebook rows padded to 256 entries. */
void launch_widen_codes(const uint8_t* packed, uint8_t* wide, uint64_t n_slots, uint32_t pq_dim,
                        uint32_t pq_bits, uint32_t n_chunks, uint32_t n_chunks8, hipStream_t stream);
void launch_pad_codebooks(const float* src, float* dst, uint64_t n_rows, uint32_t book_size, hipStream_t stream);
/** radius[l] for the `n` lists from `first_list` on: an upper bound of the length of the decoded
 *  residual (the codebook entries of a row's codes, side by side) over the list's rows. */
void launch_list_radius(const uint8_t* const* data_ptrs, const uint32_t* list_sizes, uint32_t first_list,
                        uint32_t n, uint32_t pq_dim, uint32_t pq_bits, uint32_t pq_len, const float* pq_centers,
                        bool per_subspace, float* radius, hipStream_t stream);
void launch_build_lead_plane(const uint8_t* arena, uint64_t* plane, uint64_t n_slots,
                             uint32_t n_chunks, hipStream_t stream);
constexpr uint64_t kLeadPlaneSlack = 512;  // slots past the last list that look-ahead loads of whole tiles may read
/** Persistent kernel for 8-bit codes and common shapes (scan_fast.hip); returns false when the
 *  arguments are outside what it covers.  Needs `a.desc`. */
bool scan_fast_supported(const scan_args& a);
bool launch_scan_fast(const scan_args& a, hipStream_t stream);

/** The 4-bit variant of the block kernel (pq_bits = 4, pq_dim a multiple of 32; scan_nibble.hip):
 *  same records, candidate keys and bound updates. */
bool scan_nibble_supported(const scan_args& a);
bool launch_scan_nibble(const scan_args& a, hipStream_t stream);
/** 4-bit codes with binary16 sums, two rows per lane and one wave per pair (pq_dim a multiple of 128
 *  up to 512, k <= 64, fp16 or 8-bit tables; scan_nibble_pack.hip).  k keys per pair. */
bool scan_nibble_pack_supported(const scan_args& a);
/** Table-free wave-per-pair scan for fp32 tables (8-bit codes, L2, per-subspace codebooks, pq_len 2,
 *  k <= 64): what the leading and the surviving pairs of an early stop take. */
bool scan_direct_supported(const scan_args& a);
bool launch_scan_direct(const scan_args& a, hipStream_t stream);
bool launch_scan_nibble_pack(const scan_args& a, hipStream_t stream);
/** CU-wide kernel for 8-bit codes, k <= 128 and fp16 / 8-bit tables (scan_stream.hip).  It writes
 *  several candidate groups per pair: scan_stream_keys_per_pair() is the number of keys the output
 *  buffer must hold per (query, probe) pair, 0 when the arguments are outside what it covers. */
uint32_t scan_stream_keys_per_pair(const scan_args& a);
bool launch_scan_stream(const scan_args& a, hipStream_t stream);
/** The same organisation with the table of a pair taken in slabs of 64 subspaces (scan_slab.cuh):
 *  8-bit codes, pq_dim a multiple of 32, pq_len 1, 2, 3, 4 or 8, k <= 128, fp16 / 8-bit tables. */
uint32_t scan_slab_keys_per_pair(const scan_args& a);
bool launch_scan_slab(const scan_args& a, hipStream_t stream);

/**
 * Early termination for L2 metrics, as compute_score's early stop in the reference
 * (cpp/src/neighbors/ivf_pq/detail/jit_lto_kernels/compute_score_impl.cuh:70-74): a row whose
 * partial sum over the first subspaces already exceeds the query's current k-th best score cannot
 * enter the result.  The screen kernel (scan_screen.hip) builds the lookup table of the first 16
 * subspaces only, sums the first 16-byte chunk of every row of a pair and keeps the pair only if
 * some row is still below the query's bound; surviving records are appended to `survivors`
 * (`n_survivors` counts them) and their slot is marked in `alive`.
 *
 * `n_survivors` is the first of kSurvivorWords words.  launch_order_survivors() copies the records
 * into `ordered` by length class (lists of more 64-row tiles first; its table of counts takes the
 * words from kSurvivorTable on): the persistent scan kernels hand their blocks the records in turn
 * and couple the pairs of an iteration, so records in order of length give every block the same
 * work and an iteration two pairs of the same length.
 */
constexpr uint32_t kSurvivorClasses = 256;
constexpr uint32_t kFarPairsWord    = 1;  // pairs dropped on their length alone are counted here
constexpr uint32_t kKeptPairsWord   = 2;  // launch_far_filter(): records it left for the screen
constexpr uint32_t kSurvivorTable   = 64;
constexpr uint32_t kFarBlocks       = 1024;
constexpr uint32_t kFarTable        = kSurvivorTable + 64 * kSurvivorClasses;  // its table of block counts
constexpr uint32_t kSurvivorWords   = kFarTable + kFarBlocks;
void launch_order_survivors(const pair_desc* survivors, uint32_t* n_survivors, pair_desc* ordered,
                            hipStream_t stream);

/**
 * Before the screen of an L2 search: the records of the pairs whose lists lie, row for row,
 * provably past their query's bound are left out (scan_far.hip).  `desc` are the screened pairs'
 * records, `kept` receives the others in the same order and words[count_word] their number;
 * words[kFarPairsWord] grows by the number left out.  With `alive` non-null the kept pairs' slots
 * are marked there (the search then takes them for the survivors without a screen).  The probe's fp32 coarse score comes from
 * `probe_scores` (by pair slot), or from the score matrix `score_rows` where that is null or the
 * query's byte in `from_rows` is set.  keep / slack / cap as scan_args' prune_*; eps_rel: relative
 * rounding allowance of the squared length (L2) or of the score (inner product).
 */
struct far_args {
  const pair_desc* desc;
  uint32_t n_pairs;
  pair_desc* kept;
  uint32_t* words;
  const float* probe_scores;
  const float* score_rows;
  uint32_t n_lists;
  const uint8_t* from_rows;
  const float4* center_terms;  // per list: stored |c|^2, |c_rot|^2, |R^T c_rot - c|
  const float* list_radius;
  float4* qterms;              // scratch, n_queries entries
  float keep, slack, cap, eps_rel;
  int ip;                      // 1 inner product, 2 cosine: the bound is score - |q| e - |R q| radius, less `tol` of
  float tol;                   // the entries' summed magnitudes (what the table and the sums may lose)
  uint32_t count_word;         // kKeptPairsWord, or 0 when the kept pairs are the survivors
  uint8_t* alive;              // or null
  int unordered;               // the kept records' order does not matter and words[count_word] is zero:
                               // one pass, the blocks claim their records' places as they come
};
void launch_far_filter(const far_args& f, const float* rot_q, const float* qf, uint32_t rot_dim, uint32_t dim,
                       const uint32_t* query_kth, uint32_t n_queries, const float* rotation_t, bool identity,
                       hipStream_t stream);
void launch_center_terms(const float* centers, const float* centers_rot, const float* rotation, uint32_t n_lists,
                         uint32_t dim, uint32_t dim_ext, uint32_t rot_dim, bool identity, float4* terms,
                         hipStream_t stream);
bool scan_screen_supported(const scan_args& a);
/** Bytes of each row the screen reads (8 or 16). */
uint32_t scan_screen_bytes_per_row(bool per_cluster, bool lead_plane);
/** Inner-product and cosine searches are screened on a proven lower bound of what the subspaces
 *  past the leading ones can still add; the bound's per-query part lives in `scratch`
 *  (scan_screen_scratch_bytes() bytes for the batch, 0 for L2 metrics; rewritten by every launch). */
size_t scan_screen_scratch_bytes(const scan_args& a, uint32_t n_queries);
void launch_scan_screen(const scan_args& a, const pair_desc* desc, uint32_t n_pairs,
                        pair_desc* survivors, uint32_t* n_survivors, uint8_t* alive, void* scratch,
                        hipStream_t stream);
/** query_kth[q] = min(query_kth[q], score of the k-th smallest valid key among the first `n_keys`
 *  keys of query q's candidate block (`keys_per_query` keys apart)). */
void launch_kth_bound(const unsigned long long* keys, uint32_t n_queries, uint64_t keys_per_query,
                      uint32_t n_keys, uint32_t k, uint32_t* query_kth, hipStream_t stream);

struct merge_args {
  uint32_t n_queries, n_probes, k, max_samples;
  uint32_t keys_per_pair;  // fused: candidate keys stored per (query, probe) pair
  int fused;
  int metric;
  float scaling;
  const unsigned long long* in_keys;  // fused
  const uint8_t* alive;               // fused: per pair slot, 0 = no keys were written (or null: all)
  uint8_t* redo;                      // with alive: scratch, a byte per query (null: one kernel does all)
  const uint32_t* bound;              // fused: per query, an upper bound of the final k-th key's score word (or null)
  const float* in_scores;             // non-fused
  const uint32_t* n_samples;
  const uint32_t* probes;
  const uint32_t* chunk_indices;
  const int64_t* const* inds_ptrs;
  int64_t* neighbors;  // [n_queries, k]
  float* distances;    // [n_queries, k]
  unsigned long long* out_scratch;  // k beyond kMergeLdsK: [n_queries, next_pow2(k)] keys (else null)
};
constexpr uint32_t kMergeLdsK = 8192;  // the selection's output of up to this many keys sits in LDS
void launch_merge(const merge_args& a, hipStream_t stream);

/** Exact re-ranking of candidates (refine.hip): ids and distances of the k best candidates of every
 *  query, ascending distance (descending similarity with `ip`). */
/** Ids between the two widths the refinement's interfaces take. */
void launch_widen_ids(const uint32_t* in, int64_t* out, uint64_t n, hipStream_t stream);
void launch_narrow_ids(const int64_t* in, uint32_t* out, uint64_t n, hipStream_t stream);
void launch_refine(const void* dataset, const void* queries, elem_type type,
                   const int64_t* candidates, int64_t n_rows, uint32_t n_queries, uint32_t dim,
                   uint32_t n_candidates, uint32_t k, bool ip, bool sqrt_out, int64_t* indices,
                   float* distances, hipStream_t stream);

/* list maintenance and encoding */
void launch_normalize_rows(float* x, uint64_t n_rows, uint32_t dim, hipStream_t stream);
/** counts[l] += number of labels equal to l, for l < n_bins; larger labels are skipped. */
void launch_histogram(const uint32_t* labels, uint64_t n, uint32_t n_bins, uint32_t* counts,
                      hipStream_t stream);
void launch_relocate_lists(const uint8_t* old_codes, const int64_t* old_ids, uint8_t* new_codes,
                           int64_t* new_ids, const uint64_t* old_row_offsets,
                           const uint64_t* new_row_offsets, const uint32_t* old_sizes,
                           uint32_t n_lists, uint32_t n_chunks, hipStream_t stream);
struct encode_args {
  const float* xf;  // mapped rows [n, dim]
  uint64_t n_rows;
  uint32_t dim, dim_ext, rot_dim, pq_dim, pq_len, pq_bits, n_chunks;
  int per_cluster;
  const uint32_t* labels;
  const uint32_t* perm;  // thread i encodes row perm[i] (rows grouped by list), or null: row i
  const float* centers;
  const float* rotation_t;
  int identity_rotation;
  const float* pq_centers;
  /* mode A: append into lists */
  uint32_t* cursors;          // [n_lists] next free slot per list
  uint8_t* const* data_ptrs;  // per-list code base
  int64_t* const* inds_ptrs;  // per-list id base
  const int64_t* ids;         // [n] or null
  int64_t first_id;           // used when ids is null
  /* mode B: bit-contiguous output rows */
  uint8_t* flat_codes;  // [n, ceil(pq_dim * pq_bits / 8)] or null
  float* scratch;       // [rot_dim, n] rotated residuals
};
void launch_encode(const encode_args& a, hipStream_t stream);

/** perm = the row numbers 0..n-1 grouped by label (order inside a group unspecified);
 *  `counters` holds 2 * n_lists words of scratch. */
void launch_rows_by_label(const uint32_t* labels, uint64_t n, uint32_t n_lists, uint32_t* counters,
                          uint32_t* perm, hipStream_t stream);

void launch_unpack_contiguous(const uint8_t* list_data, uint32_t n_rows, uint32_t offset,
                              uint32_t pq_dim, uint32_t pq_bits, uint8_t* out, hipStream_t stream);

/* Codes of one list outside the search (list_codes.hip).  `rows` selects rows of the list by
 * position; null: rows offset .. offset + n_rows - 1. */
/** out [n_rows, pq_dim]: one code per byte. */
void launch_unpack_codes(const uint8_t* list_data, uint32_t n_rows, uint32_t offset,
                         const uint32_t* rows, uint32_t pq_dim, uint32_t pq_bits, uint8_t* out,
                         hipStream_t stream);
/** Overwrites rows offset .. offset + n_rows - 1 of the list; `codes` holds one code per byte
 *  ([n_rows, pq_dim]) or, `contiguous`, bit strings of ceil(pq_dim * pq_bits / 8) bytes per row. */
void launch_pack_codes(uint8_t* list_data, const uint8_t* codes, bool contiguous, uint32_t n_rows,
                       uint32_t offset, uint32_t pq_dim, uint32_t pq_bits, hipStream_t stream);
/** out [n_rows, pq_dim * pq_len]: the rows decoded in the rotated space (centre + codebook entries);
 *  `book_base` is the list's codebook (per-cluster) or the first subspace's (per-subspace). */
void launch_reconstruct_rot(const uint8_t* list_data, uint32_t n_rows, uint32_t offset,
                            const uint32_t* rows, uint32_t pq_dim, uint32_t pq_bits, uint32_t pq_len,
                            const float* book_base, bool per_subspace, const float* center_rot,
                            float* out, hipStream_t stream);
/** float values back to the rows' element type (the inverse of the scaling applied on the way in). */
void launch_unmap_rows(const float* in, uint64_t n_elems, elem_type type, void* out, hipStream_t stream);

/** rotation [rot_dim, dim] on the host: the identity unless a random one is asked for or needed
 *  (rot_dim != dim): then `dim` orthonormal columns (train.cpp). */
std::vector<float> make_rotation(uint32_t rot_dim, uint32_t dim, bool force_random);

/** Gives every list room for `new_sizes[l]` rows (not less than it holds): lays the two arenas out
 *  again, moves the stored rows, and updates the host and device tables.  The device list sizes
 *  become `new_sizes` as well; rows past a list's old size are zero codes and id -1 until written.
 *  Synchronises the stream. */
void relayout_lists(const cuvs::resources& res, index_impl& ix, const std::vector<uint32_t>& new_sizes);

}  // namespace cuvs::neighbors::ivf_pq::detail
