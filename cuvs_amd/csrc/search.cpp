/*
 * Host driver of IVF-PQ search.  Validation, probe-count clamping, the max_samples bound and the
 * score / lookup-table type rules follow cuVS detail::search and ivfpq_search::fun
 * (cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:878-1048, :681-743); batching and the kernel
 * plan are this library's own (results do not depend on how queries are batched).
 */
#include "detail.hpp"
#include "tracing.hpp"

#include <algorithm>
#include <exception>
#include <mutex>
#include <cstdlib>
#include <limits>
#include <vector>

namespace cuvs {

struct resources::profile_state {
  hipEvent_t ev[7]            = {};
  unsigned long long* d_stats = nullptr;
};

void destroy_profile_state(resources::profile_state* p)
{
  if (p == nullptr) { return; }
  for (auto& e : p->ev) {
    if (e != nullptr) { (void)hipEventDestroy(e); }
  }
  if (p->d_stats != nullptr) { (void)hipFree(p->d_stats); }
  delete p;
}

}  // namespace cuvs

namespace cuvs::neighbors::ivf_pq {

namespace {

using detail::index_impl;

constexpr uint32_t kMaxFusedK = 256;   // larger k dumps all scores and selects afterwards
constexpr size_t kMaxLds      = 160 * 1024;
constexpr uint32_t kFewPairs  = 640;  // (query, probe) pairs of a batch up to which they are scanned in one plain launch
                                       // (headline index, 64 probes: 8 queries 0.082 ms; 16 queries 0.12 ms against 0.098 ms by the early stop)

/** A pointer is usable by kernels when HIP knows it as device, managed or pinned host memory
 *  (role of utils::check_pointer_residency, detail/ann_utils.cuh). */
bool device_accessible(const void* p)
{
  hipPointerAttribute_t attr;
  const hipError_t st = hipPointerGetAttributes(&attr, p);
  if (st != hipSuccess) {
    (void)hipGetLastError();  // clear the sticky error left by an unregistered host pointer
    return false;
  }
  return attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged ||
         attr.type == hipMemoryTypeHost || attr.type == hipMemoryTypeArray;
}

size_t workspace_budget(const cuvs::resources& res)
{
  if (res.workspace_borrowed()) { return res.workspace_capacity(); }
  size_t free_b = 0, total_b = 0;
  CUVS_HIP_TRY(hipMemGetInfo(&free_b, &total_b));
  // what is already cached in the workspace counts as available
  size_t budget = (free_b + res.workspace_capacity()) / 10 * 4;
  if (res.workspace_limit() != 0) { budget = std::min(budget, res.workspace_limit()); }
  return std::max(budget, size_t(64) << 20);
}

struct plan {
  uint32_t n_probes;
  uint32_t max_samples;
  bool fused;
  uint32_t batch;
  size_t per_query_bytes;
  size_t fixed_bytes;
};

size_t a256(size_t v) { return (v + 255) & ~size_t(255); }

plan make_plan(const cuvs::resources& res, const search_params& params, const index_impl& ix,
               uint32_t n_queries, uint32_t k)
{
  plan p{};
  p.n_probes = std::min<uint32_t>(params.n_probes, ix.n_lists);
  {
    // ivf_pq_search.cuh:934-940
    const int64_t ms = ((ix.accum_sorted_sizes[p.n_probes] + 127) / 128) * 128;
    CUVS_EXPECTS(ms <= int64_t(std::numeric_limits<uint32_t>::max()),
                 "The maximum sample size is too big.");
    p.max_samples = uint32_t(ms);
  }
  p.fused = k <= kMaxFusedK;
  const size_t P = p.n_probes;
  p.per_query_bytes = size_t(ix.dim) * 4 + size_t(ix.dim_ext) * 4 + size_t(ix.n_lists) * 4 +
                      size_t(ix.rot_dim) * 4 +
                      P * 4 * 3 + P * (2 * sizeof(detail::pair_desc) + 1) + 17 + P * 17 + P * 4 + 16 +
                      (p.fused ? P * k * 8 * 4 : size_t(p.max_samples) * 4) +
                      (k > detail::kMergeLdsK ? size_t(next_pow2(k)) * 8 : 0) +
                      detail::select_probes_scratch_bytes(1, uint32_t(P));
  p.fixed_bytes = a256(size_t(ix.n_lists) * 16 + 16) + 3 * 256 + size_t(512) * 8 + a256(size_t(ix.dim_ext) * 128 * 4) + a256(detail::kSelectSlackBytes) + 20 * 256;
  if (ix.coarse_fast_ok) {
    // buffers of the two-precision probe selection (the batch must fit with them)
    p.per_query_bytes += size_t(detail::coarse_fast_k_pad(ix.dim)) * 2 + size_t(detail::coarse_fast_groups(ix.n_lists)) * 4 +
                         size_t(detail::coarse_fast_cand_cap()) * 4 + 16;
    p.fixed_bytes += a256(size_t(128) * (detail::coarse_fast_k_pad(ix.dim) * 2 + 8)) + 8 * 256;
  }
  const size_t budget = workspace_budget(res);
  size_t b = budget > p.fixed_bytes ? (budget - p.fixed_bytes) / (p.per_query_bytes + 64) : 1;
  b        = std::max<size_t>(b, 1);
  b        = std::min<size_t>(b, std::max<uint32_t>(params.max_internal_batch_size, 1u));
  b        = std::min<size_t>(b, n_queries);
  // keep the pair count of a batch within uint32 indexing
  while (b > 1 && b * P >= (size_t(1) << 31)) { b /= 2; }
  // batches of equal size: 10,000 queries at a limit of 4096 run as 3 x 3334, not 4096 + 4096 + 1808
  // (a short last batch leaves most of the persistent grids' last round idle)
  const size_t n_batches = (size_t(n_queries) + b - 1) / b;
  b                      = (size_t(n_queries) + n_batches - 1) / n_batches;
  p.batch = uint32_t(b);
  return p;
}

void validate(const search_params& params, const index_impl& ix, int64_t k)
{
  // ivf_pq_search.cuh:901-923
  CUVS_EXPECTS(params.internal_distance_dtype == CUDA_R_16F ||
                 params.internal_distance_dtype == CUDA_R_32F,
               "internal_distance_dtype must be either CUDA_R_16F or CUDA_R_32F");
  CUVS_EXPECTS(params.lut_dtype == CUDA_R_16F || params.lut_dtype == CUDA_R_32F ||
                 params.lut_dtype == CUDA_R_8U,
               "lut_dtype must be CUDA_R_16F, CUDA_R_32F or CUDA_R_8U");
  CUVS_EXPECTS(k > 0, "parameter `k` in top-k must be positive.");
  CUVS_EXPECTS(k <= ix.size,
               "parameter `k` (%lld) in top-k must not be larger that the total size of the index "
               "(%lld)",
               static_cast<long long>(k), static_cast<long long>(ix.size));
  CUVS_EXPECTS(params.n_probes > 0,
               "n_probes (number of clusters to probe in the search) must be positive.");
  // ivf_pq_search.cuh:699-707
  CUVS_EXPECTS(!(params.internal_distance_dtype == CUDA_R_16F && params.lut_dtype == CUDA_R_32F),
               "Unexpected lut_dtype / internal_distance_dtype combination (%d, %d). Size of the "
               "internal_distance_dtype should be not smaller than the size of the lut_dtype.",
               int(params.lut_dtype), int(params.internal_distance_dtype));
  CUVS_EXPECTS(params.coarse_search_dtype == CUDA_R_32F || params.coarse_search_dtype == CUDA_R_16F ||
                 params.coarse_search_dtype == CUDA_R_8I,
               "Unsupported coarse_search_dtype (only CUDA_R_32F, CUDA_R_16F, and CUDA_R_8I are supported)");
}

/** Probes per query whose lists are scanned in full before the others are screened against the
 *  bound they give (2 to 16 measured no better on clustered data). */
constexpr uint32_t kLeadProbes = 1;

float scaling_factor(elem_type t)
{
  // utils::config<T>::kDivisor / utils::config<float>::kDivisor (ivf_pq_search.cuh:1043)
  return t == elem_type::u8 ? 256.0f : (t == elem_type::i8 ? 128.0f : 1.0f);
}

size_t elem_size(elem_type t) { return t == elem_type::f32 ? 4 : (t == elem_type::f16 ? 2 : 1); }

struct coarse_buffers {
  float* qt;  // [dim_ext][coarse_pad(batch)]
  float* qf;
  float* scores;
  uint32_t* probes;
  void* select_scratch = nullptr;  // beyond kSelectLdsProbes probes: where the selection writes
  // two-precision selection (null when it does not apply)
  _Float16* qh      = nullptr;
  float* qnorm      = nullptr;
  float* minima     = nullptr;
  float* thr        = nullptr;
  uint32_t* cand_count = nullptr;
  uint32_t* cand    = nullptr;
  uint8_t* fallback = nullptr;
  float* probe_scores = nullptr;  // wanted by the search: the probes' fp32 scores
};

/** The two-precision probe selection applies to fp32 coarse search and to shapes where its
 *  candidate lists stay short: about 1.4 n_probes lists per query pass the threshold, and a
 *  workgroup of the candidate pass (512 lists) holds at most 32 of them per query before the query
 *  falls back to the plain path, so n_lists >= 64 n_probes keeps the expected load near 11. */
bool coarse_fast_applies(const cuvs::resources& res, const search_params& params,
                         const index_impl& ix, uint32_t n_probes)
{
  return !res.tuning.plain_coarse && ix.coarse_fast_ok &&
         params.coarse_search_dtype == CUDA_R_32F && n_probes <= detail::coarse_fast_cand_cap() / 2 &&
         ix.n_lists >= 1024 && ix.n_lists >= 64u * n_probes && ix.dim <= detail::coarse_fast_max_dim();
}

/** Workspace bytes of the two-precision selection for a batch, and its allocation. */
size_t coarse_fast_bytes(const index_impl& ix, size_t batch)
{
  const size_t q_pad = detail::coarse_pad(uint32_t(batch));
  return a256(q_pad * detail::coarse_fast_k_pad(ix.dim) * 2) + a256(q_pad * 4) +
         a256(batch * detail::coarse_fast_groups(ix.n_lists) * 4) + a256(batch * 4) + a256(q_pad * 4) +
         a256(batch * detail::coarse_fast_cand_cap() * 4) + a256(batch + 4);
}

void alloc_coarse_fast(cuvs::resources& res, const index_impl& ix, size_t batch, coarse_buffers& b)
{
  const size_t q_pad = detail::coarse_pad(uint32_t(batch));
  b.qh         = static_cast<_Float16*>(res.workspace_alloc(q_pad * detail::coarse_fast_k_pad(ix.dim) * 2));
  b.qnorm      = static_cast<float*>(res.workspace_alloc(q_pad * 4));
  b.minima     = static_cast<float*>(res.workspace_alloc(batch * detail::coarse_fast_groups(ix.n_lists) * 4));
  b.thr        = static_cast<float*>(res.workspace_alloc(batch * 4));
  b.cand_count = static_cast<uint32_t*>(res.workspace_alloc(q_pad * 4));
  b.cand       = static_cast<uint32_t*>(res.workspace_alloc(batch * detail::coarse_fast_cand_cap() * 4));
  b.fallback   = static_cast<uint8_t*>(res.workspace_alloc(batch + 4));
}

/** mapping + centre scores + probe selection for one batch */
void run_coarse(const cuvs::resources& res, const search_params& params, const index_impl& ix,
                const void* queries, elem_type type, uint32_t nq, uint32_t n_probes,
                const coarse_buffers& b)
{
  cuvs::tracing::range scope("ivf_pq::search::select_clusters(n_probes = %u, n_queries = %u, n_lists = %u, dim = %u)",
                             n_probes, nq, ix.n_lists, ix.dim);
  hipStream_t s     = res.stream();
  const bool ip     = ix.metric == detail::DistanceType::InnerProduct ||
                  ix.metric == detail::DistanceType::CosineExpanded;
  if (b.qh != nullptr) {
    detail::coarse_fast_args a{};
    a.qf         = b.qf;  // the packing kernel maps the queries on its way
    a.queries    = queries;
    a.type       = type;
    a.n_queries  = nq;
    a.n_lists    = ix.n_lists;
    a.dim        = ix.dim;
    a.dim_ext    = ix.dim_ext;
    a.n_probes   = n_probes;
    a.ip_like    = ip;
    a.centers    = ix.centers.as<float>();
    a.ch         = ix.centers_h.as<_Float16>();
    a.cn         = ix.center_norms.as<float>();
    a.c_max      = ix.c_max;
    a.n_max      = ix.n_max;
    a.qh         = b.qh;
    a.qnorm      = b.qnorm;
    a.minima     = b.minima;
    a.thr        = b.thr;
    a.cand_count = b.cand_count;
    a.cand       = b.cand;
    a.fallback   = b.fallback;
    a.scores     = b.scores;
    a.probes     = b.probes;
    a.probe_scores = b.probe_scores;
    detail::launch_coarse_fast(a, s);
    return;
  }
  detail::launch_map_queries(queries, type, uint64_t(nq) * ix.dim, b.qf, s);
  if (params.coarse_search_dtype == CUDA_R_8I) {
    // ivf_pq_search.cuh:170-256
    detail::launch_coarse_scores_i8(b.qf, ix.centers_i8.as<uint32_t>(), nq, ix.n_lists, ix.dim, ip,
                                    b.scores, s);
    detail::launch_select_probes(b.scores, nq, ix.n_lists, n_probes, b.probes, s, nullptr, b.select_scratch);
    return;
  }
  detail::launch_map_queries_t(queries, type, nq, ix.dim, ix.dim_ext, ip, b.qt, s);
  detail::launch_coarse_scores_mfma(b.qt, ix.centers_t.as<float>(), nq, ix.n_lists, ix.dim_ext, ip,
                                    params.coarse_search_dtype == CUDA_R_16F, b.scores, s);
  detail::launch_select_probes(b.scores, nq, ix.n_lists, n_probes, b.probes, s, nullptr, b.select_scratch);
}

}  // namespace

void select_clusters(cuvs::resources const& res_c,
                     const search_params& params,
                     const index<int64_t>& idx,
                     const void* queries,
                     elem_type type,
                     int64_t n_queries,
                     uint32_t* clusters_to_probe)
{
  auto& res      = const_cast<cuvs::resources&>(res_c);
  const auto& ix = *idx.impl();
  CUVS_EXPECTS(params.n_probes > 0,
               "n_probes (number of clusters to probe in the search) must be positive.");
  CUVS_EXPECTS(params.coarse_search_dtype == CUDA_R_32F || params.coarse_search_dtype == CUDA_R_16F ||
                 params.coarse_search_dtype == CUDA_R_8I,
               "Unsupported coarse_search_dtype (only CUDA_R_32F, CUDA_R_16F, and CUDA_R_8I are supported)");
  CUVS_EXPECTS(device_accessible(queries) && device_accessible(clusters_to_probe),
               "all pointers must be accessible from the device.");
  const uint32_t P       = std::min<uint32_t>(params.n_probes, ix.n_lists);
  const size_t per_query = size_t(ix.dim) * 4 + size_t(ix.dim_ext) * 4 + size_t(ix.n_lists) * 4 + 64;
  size_t batch           = std::max<size_t>(1, workspace_budget(res) / per_query);
  batch                  = std::min<size_t>(batch, size_t(n_queries));
  batch                  = std::min<size_t>(batch, 65535u * 64u);
  res.reset_workspace();
  const size_t qt_bytes = size_t(ix.dim_ext) * detail::coarse_pad(uint32_t(batch)) * 4;
  const bool fast       = coarse_fast_applies(res, params, ix, P);
  res.reserve_workspace(a256(batch * ix.dim * 4) + a256(qt_bytes) +
                        a256(batch * size_t(ix.n_lists) * 4 + detail::kSelectSlackBytes) + 1024 +
                        (fast ? coarse_fast_bytes(ix, batch) : 0));
  coarse_buffers b{};
  b.qt     = static_cast<float*>(res.workspace_alloc(qt_bytes));
  b.qf     = static_cast<float*>(res.workspace_alloc(batch * ix.dim * 4));
  b.scores = static_cast<float*>(
    res.workspace_alloc(batch * size_t(ix.n_lists) * 4 + detail::kSelectSlackBytes));
  if (fast) { alloc_coarse_fast(res, ix, batch, b); }
  for (int64_t q0 = 0; q0 < n_queries; q0 += int64_t(batch)) {
    const uint32_t nq = uint32_t(std::min<int64_t>(int64_t(batch), n_queries - q0));
    b.probes          = clusters_to_probe + q0 * P;
    run_coarse(res, params, ix,
               static_cast<const char*>(queries) + size_t(q0) * ix.dim * elem_size(type), type, nq,
               P, b);
  }
  res.reset_workspace();
}

namespace {
/** The search of one run of queries on one handle: its internal batches one after the other. */
void search_one(cuvs::resources const& res_c,
                const search_params& params,
                const index<int64_t>& idx,
                const void* queries,
                elem_type type,
                int64_t n_queries,
                int64_t query_dim,
                int64_t* neighbors,
                float* distances,
                int64_t k64,
                const cuvs::neighbors::filtering::base_filter& sample_filter);
}  // namespace

/**
 * Results do not depend on how the queries are batched, and `max_internal_batch_size` (4096 unless
 * the caller says otherwise) makes three batches of 10,000 queries, each a third as efficient on
 * its launches' fixed costs and tails.  So the batches of one call run side by side: the queries
 * are split at batch boundaries into up to four runs, the first on the handle's stream and
 * workspace, the others on streams and workspaces of the handle's own, which start after what the
 * handle's stream holds at the call and which the handle's stream waits for before it goes on
 * (10,000 queries of the headline workload at the default batch size: 1.43 -> 1.16 ms).  Not under
 * stream capture, with stage profiling, on a borrowed workspace or with a workspace pool.
 */
void search(cuvs::resources const& res_c,
            const search_params& params,
            const index<int64_t>& idx,
            const void* queries,
            elem_type type,
            int64_t n_queries,
            int64_t query_dim,
            int64_t* neighbors,
            float* distances,
            int64_t k64,
            const cuvs::neighbors::filtering::base_filter& sample_filter)
{
  auto& res         = const_cast<cuvs::resources&>(res_c);
  const int64_t mb  = std::max<int64_t>(int64_t(params.max_internal_batch_size), 1);
  int ways          = 1;
  int64_t per_batch = 0;
  if (n_queries > mb && !res.tuning.serial_batches && !res.profiling && !res.workspace_borrowed() &&
      res.workspace_pool() == nullptr && idx.impl() != nullptr && k64 > 0 && queries != nullptr &&
      neighbors != nullptr && distances != nullptr) {
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(res.stream(), &capture) != hipSuccess) {
      (void)hipGetLastError();
      capture = hipStreamCaptureStatusActive;  // nothing is known about the stream: stay on it
    }
    if (capture == hipStreamCaptureStatusNone) {
      const int64_t n_batches = (n_queries + mb - 1) / mb;
      per_batch               = (n_queries + n_batches - 1) / n_batches;
      ways                    = int(std::min<int64_t>(n_batches, 1 + cuvs::resources::kMaxSideHandles));
      for (int w = 1; w < ways; w++) {
        if (res.side(w - 1) == nullptr) { ways = 1; }
      }
    }
  }
  if (ways == 1) {
    search_one(res, params, idx, queries, type, n_queries, query_dim, neighbors, distances, k64, sample_filter);
    return;
  }
  const auto& ix = *idx.impl();
  if (ix.derived_stale.load()) {
    // (as in search_one: before the side streams branch off)
    std::lock_guard<std::mutex> guard(ix.derived_mu);
    if (ix.derived_stale.load()) { const_cast<index_impl&>(ix).rebuild_lead_plane(res.stream()); }
  }
  const int64_t n_batches = (n_queries + per_batch - 1) / per_batch;
  auto run_begin = [&](int w) { return std::min<int64_t>(n_queries, (int64_t(w) * n_batches / ways) * per_batch); };
  res.fork_sides(ways - 1);
  std::exception_ptr failure;
  for (int w = 0; w < ways && !failure; w++) {
    const int64_t q0 = run_begin(w), q1 = run_begin(w + 1);
    if (q1 <= q0) { continue; }
    cuvs::resources& r = w == 0 ? res : *res.side(w - 1);
    try {
      search_one(r, params, idx, static_cast<const char*>(queries) + size_t(q0) * size_t(query_dim) * elem_size(type),
                 type, q1 - q0, query_dim, neighbors + q0 * k64, distances + q0 * k64, k64, sample_filter);
    } catch (...) {
      failure = std::current_exception();  // the first run checks the arguments: nothing is queued on a side stream then
    }
  }
  res.join_sides(ways - 1);
  if (failure) { std::rethrow_exception(failure); }
}

namespace {
void search_one(cuvs::resources const& res_c,
                const search_params& params,
                const index<int64_t>& idx,
                const void* queries,
                elem_type type,
                int64_t n_queries,
                int64_t query_dim,
                int64_t* neighbors,
                float* distances,
                int64_t k64,
                const cuvs::neighbors::filtering::base_filter& sample_filter)
{
  auto& res      = const_cast<cuvs::resources&>(res_c);
  const auto& ix = *idx.impl();

  const uint32_t* filter_bits = nullptr;
  int64_t filter_nbits        = 0;
  if (dynamic_cast<const filtering::none_sample_filter*>(&sample_filter) == nullptr) {
    auto* bf = dynamic_cast<const filtering::bitset_filter*>(&sample_filter);
    CUVS_EXPECTS(bf != nullptr, "Unsupported sample filter type");  // ivf_pq_search.cuh:1126-1133
    filter_bits  = bf->bits;
    filter_nbits = bf->n_bits;
    CUVS_EXPECTS(filter_bits != nullptr && device_accessible(filter_bits),
                 "the filter bitset must be accessible from the device.");
  }

  // ivf_pq_search.cuh:1088-1096
  CUVS_EXPECTS(query_dim == int64_t(ix.dim),
               "Number of query dimensions should equal number of dimensions in the index.");
  validate(params, ix, k64);
  if (n_queries == 0) { return; }
  CUVS_EXPECTS(n_queries <= int64_t(std::numeric_limits<uint32_t>::max()), "too many queries");
  CUVS_EXPECTS(device_accessible(queries) && device_accessible(neighbors) &&
                 device_accessible(distances),
               "all pointers must be accessible from the device.");

  if (ix.derived_stale.load()) {
    // list memory was written through a bare pointer (codepacker::pack on one of the index's list
    // buffers): the copies the kernels read instead of the lists follow before anything is searched
    std::lock_guard<std::mutex> guard(ix.derived_mu);
    if (ix.derived_stale.load()) { const_cast<index_impl&>(ix).rebuild_lead_plane(res.stream()); }
  }

  const uint32_t k  = uint32_t(k64);
  cuvs::tracing::range search_scope("ivf_pq::search(n_queries = %u, n_probes = %u, k = %u, dim = %u)",
                                    uint32_t(n_queries), params.n_probes, k, ix.dim);
  const plan pl     = make_plan(res, params, ix, uint32_t(n_queries), k);
  const uint32_t P  = pl.n_probes;
  uint32_t Qb       = pl.batch;
  hipStream_t s     = res.stream();

  detail::scan_args sa{};
  sa.n_probes     = P;
  sa.k            = k;
  sa.max_samples  = pl.max_samples;
  sa.rot_dim      = ix.rot_dim;
  sa.pq_dim       = ix.pq_dim;
  sa.pq_len       = ix.pq_len;
  sa.pq_bits      = ix.pq_bits;
  sa.metric       = int(ix.metric);
  sa.per_cluster  = ix.codebook_kind == codebook_gen::PER_CLUSTER;
  sa.lut_dtype    = params.lut_dtype;
  sa.out_half     = params.internal_distance_dtype == CUDA_R_16F;
  sa.fused        = pl.fused;
  sa.centers_rot  = ix.centers_rot.as<float>();
  sa.pq_centers   = ix.pq_centers.as<float>();
  sa.data_ptrs    = ix.data_ptrs.as<const uint8_t*>();
  sa.lead_plane   = ix.lead_plane.bytes != 0 ? ix.lead_plane.as<uint64_t>() : nullptr;
  sa.inds_ptrs    = ix.inds_ptrs.as<const int64_t*>();
  sa.list_sizes   = ix.list_sizes.as<uint32_t>();
  sa.mean_list_rows = uint32_t(std::min<uint64_t>(uint64_t(ix.size) / std::max<uint32_t>(ix.n_lists, 1u), 0xFFFFFFFFull));
  sa.filter_bits  = filter_bits;
  sa.filter_nbits = filter_nbits;
  if ((ix.metric == detail::DistanceType::L2Expanded || ix.metric == detail::DistanceType::L2SqrtExpanded) &&
      ix.list_radius.bytes == sizeof(float) * ix.n_lists) {
    // what the computed sum of a row's entries can lose against exact arithmetic: the table's
    // rounding (binary16 to nearest; the unsigned 8-bit type truncates to 3 fraction bits and
    // flushes entries below 2^-15, and saturates near 1.2e5), then pq_dim additions if the sums
    // are binary16 (each rounds by at most 2^-11 of a partial sum that only grows)
    double lose  = params.lut_dtype == CUDA_R_32F ? 1e-5 : (params.lut_dtype == CUDA_R_16F ? 1.0 / 1024 : 0.07);
    double slack = params.lut_dtype == CUDA_R_8U ? double(ix.pq_dim) / 16384.0 : double(ix.pq_dim) * 1e-7;
    if (sa.out_half) { lose += double(ix.pq_dim) / 2048.0 + 1.0 / 1024; }
    if (lose < 0.5) {
      sa.list_radius = ix.list_radius.as<float>();
      sa.prune_keep  = float(1.0 - lose);
      sa.prune_slack = float(slack);
      sa.prune_cap   = params.lut_dtype == CUDA_R_8U ? 1.0e5f : std::numeric_limits<float>::infinity();
    }
  }
  if (ix.pq_bits != 8 && ix.pq_bits != 4) { sa.lead_plane = nullptr; }
  if (ix.wide() && !res.tuning.generic_scan) {
    // 5 - 7 bit codes: the byte-wide copy of the lists, if one of the 8-bit kernels takes the shape
    detail::scan_args w = sa;
    w.pq_bits    = 8;
    w.pq_centers = ix.pq_centers8.as<float>();
    w.data_ptrs  = ix.data_ptrs8.as<const uint8_t*>();
    w.lead_plane = ix.lead_plane.bytes != 0 ? ix.lead_plane.as<uint64_t>() : nullptr;
    if ((detail::scan_lds_bytes(w) <= kMaxLds &&
         (detail::scan_stream_keys_per_pair(w) != 0 || detail::scan_fast_supported(w))) ||
        detail::scan_slab_keys_per_pair(w) != 0) {
      sa = w;
    }
  }
  // the CU-wide kernels: a pair's whole table in LDS for the shapes scan_stream.hip has, else (any
  // pq_dim that is a multiple of 32) the table in slabs
  sa.fused = pl.fused;
  const uint32_t stream_kpp = res.tuning.generic_scan ? 0u : detail::scan_stream_keys_per_pair(sa);
  // fp32 tables: the table-free kernel where it has the shape (it also beats a table in slabs on
  // the lists of a few hundred rows its shapes come with), else the slab kernel
  const bool direct_scan    = !res.tuning.generic_scan && detail::scan_direct_supported(sa);
  const uint32_t slab_kpp   = res.tuning.generic_scan || stream_kpp != 0 || direct_scan ? 0u : detail::scan_slab_keys_per_pair(sa);
  // a table too large for LDS goes to global memory (8-bit codes, generic kernel)
  const bool global_lut = slab_kpp == 0 && detail::scan_lds_bytes(sa) > kMaxLds;
  if (global_lut) {
    CUVS_EXPECTS(sa.pq_bits == 8,
                 "the lookup table (pq_dim = %u, pq_bits = %u, lut_dtype = %d) needs %zu bytes of LDS, "
                 "more than the %zu available; use a smaller lut_dtype",
                 ix.pq_dim, ix.pq_bits, int(params.lut_dtype), detail::scan_lds_bytes(sa), kMaxLds);
  }
  const size_t global_lut_bytes =
    global_lut ? a256(detail::scan_lut_bytes(sa)) * detail::scan_global_lut_blocks() : 0;

  /* workspace carve-up for one batch */
  res.reset_workspace();
  const bool fast_coarse = coarse_fast_applies(res, params, ix, P);
  auto bytes_for = [&](uint32_t batch) {
    return pl.fixed_bytes + size_t(batch) * (pl.per_query_bytes + 64) + 16 * 256 + global_lut_bytes +
           a256(detail::kSurvivorWords * sizeof(uint32_t)) +
           (fast_coarse ? coarse_fast_bytes(ix, batch) : 0) + a256(detail::scan_screen_scratch_bytes(sa, batch));
  };
  if (res.workspace_borrowed()) {
    // a fixed workspace: the largest internal batch that fits it (results do not depend on how the
    // queries are batched); only a single query that does not fit is refused
    while (Qb > 1 && bytes_for(Qb) > res.workspace_capacity()) { Qb -= (Qb + 7) / 8; }
    if (Qb > 1) {
      const uint32_t n_batches = uint32_t((n_queries + Qb - 1) / Qb);
      Qb                       = uint32_t((n_queries + n_batches - 1) / n_batches);
    }
  }
  const size_t screen_scratch_bytes = a256(detail::scan_screen_scratch_bytes(sa, Qb));
  const size_t workspace_bytes      = bytes_for(Qb);
  CUVS_EXPECTS(!res.workspace_borrowed() || workspace_bytes <= res.workspace_capacity(),
               "one query (n_probes = %u, k = %u, n_lists = %u) needs %zu bytes of workspace; the fixed "
               "workspace of this call holds %zu",
               P, k, ix.n_lists, workspace_bytes, res.workspace_capacity());
  res.reserve_workspace(workspace_bytes);
  auto* qt        = static_cast<float*>(
    res.workspace_alloc(size_t(ix.dim_ext) * detail::coarse_pad(Qb) * 4));
  auto* qf        = static_cast<float*>(res.workspace_alloc(size_t(Qb) * ix.dim * 4));
  auto* scores    = static_cast<float*>(
    res.workspace_alloc(size_t(Qb) * ix.n_lists * 4 + detail::kSelectSlackBytes));
  auto* rot_q     = static_cast<float*>(res.workspace_alloc(size_t(Qb) * ix.rot_dim * 4));
  auto* probes    = static_cast<uint32_t*>(res.workspace_alloc(size_t(Qb) * P * 4));
  auto* chunk     = static_cast<uint32_t*>(res.workspace_alloc(size_t(Qb) * P * 4));
  auto* order     = static_cast<uint32_t*>(res.workspace_alloc(size_t(Qb) * P * 4));
  auto* n_samples = static_cast<uint32_t*>(res.workspace_alloc(size_t(Qb) * 4));
  auto* kth       = static_cast<uint32_t*>(res.workspace_alloc(size_t(Qb) * 4));
  auto* counters  = static_cast<uint32_t*>(res.workspace_alloc(size_t(ix.n_lists) * 16 + 16));
  coarse_buffers cb{qt, qf, scores, probes};
  if (detail::select_probes_scratch_bytes(Qb, P) != 0) {
    cb.select_scratch = res.workspace_alloc(detail::select_probes_scratch_bytes(Qb, P));
  }
  if (fast_coarse) { alloc_coarse_fast(res, ix, Qb, cb); }
  detail::pair_desc* desc = nullptr;
  unsigned long long* keys = nullptr;
  float* all_scores        = nullptr;
  sa.fused                 = pl.fused;
  if (global_lut) { sa.global_lut = res.workspace_alloc(global_lut_bytes); }
  const bool generic_only  = res.tuning.generic_scan || global_lut;
  const uint32_t quad_kpp  = generic_only ? 0u : (stream_kpp != 0 ? stream_kpp : slab_kpp);
  const bool nibble_scan   = !generic_only && detail::scan_nibble_supported(sa);
  const bool fast_scan     = !generic_only && (quad_kpp != 0 || detail::scan_fast_supported(sa) || nibble_scan ||
                                               detail::scan_direct_supported(sa));
  const uint32_t kpp       = quad_kpp != 0 ? quad_kpp : k;  // candidate keys stored per pair
  // byte codes of a shape no specialised kernel takes (pq_dim beyond 64): the generic kernel scans
  // the leading and the surviving pairs of an early stop as a subset of the pairs
  // (also nibble codes outside the wave-per-pair kernel's shapes)
  // (a table in global memory included: the generic kernel's bounded grid walks the subset as well)
  const bool generic_subset = !res.tuning.generic_scan && sa.fused &&
                              ((!fast_scan && (sa.pq_bits == 8 || sa.pq_bits == 4)) ||
                               (sa.pq_bits == 4 && !detail::scan_nibble_pack_supported(sa)));
  if (fast_scan || generic_subset) {
    desc = static_cast<detail::pair_desc*>(res.workspace_alloc(size_t(Qb) * P * sizeof(detail::pair_desc)));
  }
  // L2 early stop: lists of the leading probes in full, the others screened on their first chunk
  // A batch of a few thousand pairs is over in one or two rounds of the persistent scan grid:
  // the early stop's extra launches and the grouping of the pairs by list would cost more than
  // they save (the reference skips the grouping when lists are rarely shared,
  // expected_probe_coresidency, ivf_pq_search.cuh:353-373).
  const bool few_pairs       = uint64_t(Qb) * P <= kFewPairs;
  bool early_stop = (fast_scan || generic_subset) && !few_pairs && P > kLeadProbes && P <= 8192 &&
                    detail::scan_screen_supported(sa) && res.tuning.early_stop != 1;
  // In the automatic mode the index remembers whether the screen pays on its data: where it kept
  // most pairs the last time it ran with these parameters, this search scans plainly.
  // L2: pairs whose lists lie provably past their query's bound are left out before the screen,
  // from the probe selection's own fp32 scores (scan_far.hip)
  // (inner product: the same from the score itself; what the computed sum may lose is then relative
  // to the entries' magnitudes: the table's rounding (the signed 8-bit type keeps two fraction
  // bits), fp32 additions, and pq_dim binary16 additions where the sums are binary16)
  const bool cosine_metric = ix.metric == detail::DistanceType::CosineExpanded;
  double ip_tol = params.lut_dtype == CUDA_R_32F ? 2e-5 : (params.lut_dtype == CUDA_R_16F ? 1.0 / 1024 + 2e-5 : 0.3);
  if (sa.out_half) { ip_tol += double(ix.pq_dim) / 2048.0 + 1.0 / 1024; }
  const bool far_ip = (ix.metric == detail::DistanceType::InnerProduct || cosine_metric) && ip_tol < 0.5 &&
                      ix.list_radius.bytes == sizeof(float) * ix.n_lists;
  const bool far_possible = (sa.prune_keep > 0.0f || far_ip) && params.coarse_search_dtype == CUDA_R_32F &&
                            ix.rotation_bounded && ix.center_terms.bytes == sizeof(float4) * ix.n_lists;
  bool skip_screen    = false;  // what that leaves over is scanned in full without a screening launch
  bool observe_screen = false;
  if (early_stop && res.tuning.early_stop == 0 && ix.feedback.host != nullptr) {
    auto& fb = ix.feedback;
    std::lock_guard<std::mutex> guard(fb.mu);
    // while a stream captures, an event query invalidates the capture: the verdict stays as it is
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    CUVS_HIP_TRY(hipStreamIsCapturing(s, &capture));
    // (another thread's capture in the global mode would be invalidated by the query as well: the
    // query runs with this thread's capture mode relaxed)
    if (capture == hipStreamCaptureStatusNone) {
      hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
      CUVS_HIP_TRY(hipThreadExchangeStreamCaptureMode(&mode));
      fb.collect();
      CUVS_HIP_TRY(hipThreadExchangeStreamCaptureMode(&mode));
    }
    // (The generic kernel and the slab kernel on rows of several slabs keep the three launches even
    // then: what the leading pairs give them is a bound from a pair's first row on, which their
    // exits inside a long row live on; the screen of 8 bytes a row is a small fraction of their time.)
    const bool long_rows = slab_kpp != 0 && sa.pq_dim > 64;
    auto* verdict = fb.find(P, k);
    if (verdict != nullptr && verdict->off && !generic_subset && !long_rows) {
      verdict->plain_searches += 1;
      if (verdict->plain_searches % detail::screen_feedback::kScreenRecheck != 0) { early_stop = false; }
    }
    if (early_stop && far_possible && verdict != nullptr && !verdict->off && verdict->screen_off) {
      // the screening kernel kept most of what it was given the last time: every 64th search tries it again
      verdict->unscreened_searches += 1;
      skip_screen = verdict->unscreened_searches % detail::screen_feedback::kScreenRecheck != 0;
    }
    observe_screen = early_stop && !skip_screen && capture == hipStreamCaptureStatusNone;
    if (observe_screen && verdict != nullptr && !verdict->off && !verdict->screen_off) {
      // (a search that tries the screen again after a verdict against it is always observed)
      observe_screen = verdict->screened_searches % detail::screen_feedback::kObserveEvery == 0;
      verdict->screened_searches += 1;
    }
  }
  const uint32_t lead          = early_stop ? kLeadProbes : P;
  void* sort_scratch = few_pairs ? nullptr
                                 : res.workspace_alloc(detail::order_pairs_scratch_bytes(Qb * P, P, ix.n_lists, lead));
  detail::pair_desc* survivors = nullptr;
  uint8_t* alive               = nullptr;
  uint32_t* n_survivors        = nullptr;
  uint8_t* merge_redo          = nullptr;
  void* screen_scratch         = nullptr;
  if (early_stop) {
    survivors   = static_cast<detail::pair_desc*>(res.workspace_alloc(size_t(Qb) * P * sizeof(detail::pair_desc)));
    alive       = static_cast<uint8_t*>(res.workspace_alloc(size_t(Qb) * P));
    n_survivors = static_cast<uint32_t*>(res.workspace_alloc(detail::kSurvivorWords * sizeof(uint32_t)));
    merge_redo  = static_cast<uint8_t*>(res.workspace_alloc(size_t(Qb)));
    if (screen_scratch_bytes != 0) { screen_scratch = res.workspace_alloc(screen_scratch_bytes); }
  }
  const bool far_filter = early_stop && far_possible;
  float4* far_qterms    = nullptr;
  if (far_filter) {
    far_qterms = static_cast<float4*>(res.workspace_alloc(size_t(Qb) * sizeof(float4)));
    if (fast_coarse) { cb.probe_scores = static_cast<float*>(res.workspace_alloc(size_t(Qb) * P * 4)); }
  }
  // k beyond what the merge's LDS holds: its selection writes into global memory
  unsigned long long* merge_scratch = nullptr;
  if (k > detail::kMergeLdsK) {
    merge_scratch = static_cast<unsigned long long*>(res.workspace_alloc(size_t(Qb) * next_pow2(k) * 8));
  }
  if (pl.fused) {
    keys = static_cast<unsigned long long*>(res.workspace_alloc(size_t(Qb) * P * kpp * 8));
  } else {
    all_scores = static_cast<float*>(res.workspace_alloc(size_t(Qb) * pl.max_samples * 4));
  }

  /* profiling state */
  const bool prof = res.profiling && !res.workspace_borrowed();  // the profile allocates
  unsigned long long* d_stats = nullptr;
  if (prof) {
    if (res.prof == nullptr) {
      res.prof = new cuvs::resources::profile_state();
      for (auto& e : res.prof->ev) { CUVS_HIP_TRY(hipEventCreate(&e)); }
      CUVS_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&res.prof->d_stats), size_t(detail::kStatSlots) * 32));
    }
    d_stats = res.prof->d_stats;
    detail::launch_fill_u32(reinterpret_cast<uint32_t*>(d_stats), 0, detail::kStatSlots * 8, s);
    res.last_profile           = cuvs::search_profile{};
    res.last_profile.n_queries = uint32_t(n_queries);
    res.last_profile.n_probes  = P;
    res.last_profile.k         = k;
  }
  auto mark = [&](int i) {
    if (prof) { CUVS_HIP_TRY(hipEventRecord(res.prof->ev[i], s)); }
  };

  const bool cosine = ix.metric == detail::DistanceType::CosineExpanded;
  // the leading pairs run from long lists to short ones
  const uint32_t* list_rank = ix.list_rank.as<uint32_t>();
  for (int64_t q0 = 0; q0 < n_queries; q0 += Qb) {
    const uint32_t nq = uint32_t(std::min<int64_t>(Qb, n_queries - q0));
    const void* qptr  = static_cast<const char*>(queries) + size_t(q0) * ix.dim * elem_size(type);

    cuvs::tracing::range batch_scope("ivf_pq::search-batch(queries: %u - %u)", uint32_t(q0), uint32_t(q0) + nq);
    detail::pair_desc* screen_out = survivors;  // where the screen's survivors are, as it appended them
    mark(0);
    run_coarse(res, params, ix, qptr, type, nq, P, cb);
    mark(1);
    cuvs::tracing::range worker_scope("ivf_pq::search-worker(n_queries = %u, n_probes = %u, k = %u, dim = %u)", nq, P,
                                      k, ix.dim);
    // an identity rotation of fp32 operands leaves the mapped queries as they are
    const bool rotate = !(ix.rotation_is_identity && ix.rot_dim == ix.dim && !cosine &&
                          params.coarse_search_dtype == CUDA_R_32F);
    if (rotate) {
      detail::launch_rotate(qf, ix.rotation_t.as<float>(), nq, ix.dim, ix.rot_dim,
                            ix.rotation_is_identity, cosine, params.coarse_search_dtype, rot_q, s);
    }
    detail::launch_chunk_indices(ix.list_sizes.as<uint32_t>(), probes, nq, P,
                                 ix.n_chunks * kIndexGroupVecLen, chunk, n_samples, d_stats, lead,
                                 pl.fused ? kth : nullptr, n_survivors, 2, s);
    detail::launch_order_pairs(probes, chunk, sa.data_ptrs,
                               ix.inds_ptrs.as<const int64_t*>(), ix.ids_arena.as<int64_t>(), nq * P, P,
                               ix.n_lists, counters, sort_scratch, order, desc, lead, alive, few_pairs, list_rank, s);
    mark(2);

    {
    cuvs::tracing::range scan_scope("ivf_pq::search-worker::scan");
    sa.n_queries     = nq;
    sa.rot_q         = rotate ? rot_q : qf;
    sa.probes        = probes;
    sa.chunk_indices = chunk;
    sa.pair_order    = order;
    sa.query_kth     = kth;
    sa.out_keys      = keys;
    sa.out_scores    = all_scores;
    sa.desc        = desc;
    sa.n_pairs     = nq * P;
    sa.n_pairs_dev = nullptr;
    // the kernel that scans pairs in full (the launchers return false for arguments they do not
    // cover); which one it was goes into the profile
    uint32_t scan_kernel_id = cuvs::scan_kernel_generic;
    auto full_scan = [&](bool subset) {
      if (subset && generic_subset) {
        sa.subset = 1;
        detail::launch_scan(sa, s);
        sa.subset      = 0;
        scan_kernel_id = cuvs::scan_kernel_generic;
        return;
      }
      if (fast_scan) {
        if (slab_kpp != 0) {
          if (detail::launch_scan_slab(sa, s)) { scan_kernel_id = cuvs::scan_kernel_slab; return; }
        } else if (quad_kpp != 0) {
          if (detail::launch_scan_stream(sa, s)) { scan_kernel_id = cuvs::scan_kernel_stream; return; }
        } else if (sa.pq_bits == 4) {
          if (detail::launch_scan_nibble_pack(sa, s)) { scan_kernel_id = cuvs::scan_kernel_nibble_pack; return; }
          if (!subset && detail::launch_scan_nibble(sa, s)) { scan_kernel_id = cuvs::scan_kernel_nibble; return; }
        } else {
          if (direct_scan && detail::launch_scan_direct(sa, s)) { scan_kernel_id = cuvs::scan_kernel_direct; return; }
          if (detail::launch_scan_fast(sa, s)) { scan_kernel_id = cuvs::scan_kernel_fast; return; }
        }
      }
      CUVS_EXPECTS(!subset, "scan kernel launch failed");
      detail::launch_scan(sa, s);
      scan_kernel_id = cuvs::scan_kernel_generic;
    };
    if (early_stop) {
      // 1. the leading probes' lists in full: candidates and a first bound per query
      sa.n_pairs    = nq * lead;
      sa.rare_exits = 1;  // no bound yet here, and the screen's survivors mostly stay under theirs
      full_scan(true);
      detail::launch_kth_bound(keys, nq, uint64_t(P) * kpp, lead * kpp, k, kth, s);
      mark(5);
      // 2. every other pair on its first chunk only
      detail::pair_desc* screened = desc + size_t(nq) * lead;
      const uint32_t n_screened   = nq * (P - lead);
      if (far_filter) {
        // the pairs worth screening go to the survivors' buffer, the screen's survivors where the
        // screened pairs' records were, and the ordered survivors back again
        detail::far_args f{};
        f.desc         = screened;
        f.n_pairs      = n_screened;
        f.kept         = survivors;
        f.words        = n_survivors;
        f.probe_scores = cb.probe_scores;
        f.score_rows   = scores;
        f.n_lists      = ix.n_lists;
        f.from_rows    = cb.probe_scores != nullptr ? cb.fallback : nullptr;
        f.center_terms = ix.center_terms.as<float4>();
        f.list_radius  = ix.list_radius.as<float>();
        f.ip           = far_ip ? (cosine_metric ? 2 : 1) : 0;
        f.tol          = float(ip_tol);
        f.qterms       = far_qterms;
        f.keep         = sa.prune_keep;
        f.slack        = cosine_metric ? (sa.out_half ? 2e-3f : 2e-6f) : sa.prune_slack;
        f.cap          = sa.prune_cap;
        f.eps_rel      = float(ix.dim + ix.rot_dim + 16) * 1.2e-7f;
        f.count_word   = skip_screen ? 0u : detail::kKeptPairsWord;
        f.alive        = skip_screen ? alive : nullptr;
        f.unordered    = skip_screen ? 1 : 0;  // (the survivors are put in order of length next)
        detail::launch_far_filter(f, sa.rot_q, qf, ix.rot_dim, ix.dim, kth, nq, ix.rotation_t.as<float>(),
                                  ix.rotation_is_identity && ix.rot_dim == ix.dim, s);
        if (!skip_screen) {
          // (the screening kernels' own look at a pair's length would repeat the same test)
          const float keep    = sa.prune_keep;
          sa.prune_keep       = 0.0f;
          sa.screen_pairs_dev = n_survivors + detail::kKeptPairsWord;
          detail::launch_scan_screen(sa, survivors, n_screened, screened, n_survivors, alive, screen_scratch, s);
          sa.screen_pairs_dev = nullptr;
          sa.prune_keep       = keep;
          screen_out          = screened;
        }
      } else {
        detail::launch_scan_screen(sa, screened, n_screened, survivors, n_survivors, alive, screen_scratch, s);
      }
      if (observe_screen) {
        // the survivor count follows the search to the host, for the searches after this one
        observe_screen = false;
        auto& fb       = ix.feedback;
        std::lock_guard<std::mutex> guard(fb.mu);
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        CUVS_HIP_TRY(hipThreadExchangeStreamCaptureMode(&mode));
        fb.collect();
        CUVS_HIP_TRY(hipThreadExchangeStreamCaptureMode(&mode));
        if (!fb.pending) {
          CUVS_HIP_TRY(hipMemcpyAsync(fb.host, n_survivors, 8, hipMemcpyDeviceToHost, s));
          fb.pending_far    = far_filter;
          CUVS_HIP_TRY(hipEventRecord(fb.landed, s));
          fb.pending        = true;
          fb.pending_pairs  = uint64_t(nq) * (P - lead);
          fb.pending_probes = P;
          fb.pending_k      = uint32_t(k);
        }
      }
      mark(6);
      // 3. the pairs still in play, in full, from long lists to short ones (the records of the
      // screened pairs are done with: the ordered ones take their place)
      detail::pair_desc* ordered = screen_out == survivors ? screened : survivors;
      detail::launch_order_survivors(screen_out, n_survivors, ordered, s);
      sa.desc        = ordered;
      sa.n_pairs     = 0;
      sa.n_pairs_dev = n_survivors;
      full_scan(true);
    } else {
      full_scan(false);
    }
    if (prof) { res.last_profile.scan_kernel = scan_kernel_id; }
    }
    mark(3);

    cuvs::tracing::range merge_scope("ivf_pq::search-worker::merge");
    detail::merge_args ma{};
    ma.n_queries     = nq;
    ma.n_probes      = P;
    ma.k             = k;
    ma.max_samples   = pl.max_samples;
    ma.fused         = pl.fused;
    ma.keys_per_pair = kpp;
    ma.metric        = int(ix.metric);
    ma.scaling       = scaling_factor(type);
    ma.in_keys       = keys;
    ma.alive         = alive;
    ma.redo          = merge_redo;
    ma.bound         = pl.fused ? kth : nullptr;
    ma.in_scores     = all_scores;
    ma.n_samples     = n_samples;
    ma.probes        = probes;
    ma.chunk_indices = chunk;
    ma.inds_ptrs     = ix.inds_ptrs.as<const int64_t*>();
    ma.neighbors     = neighbors + q0 * k;
    ma.distances     = distances + q0 * k;
    ma.out_scratch   = merge_scratch;
    detail::launch_merge(ma, s);
    mark(4);

    if (prof) {
      CUVS_HIP_TRY(hipEventSynchronize(res.prof->ev[4]));
      float ms[4] = {0, 0, 0, 0};
      for (int i = 0; i < 4; i++) {
        CUVS_HIP_TRY(hipEventElapsedTime(&ms[i], res.prof->ev[i], res.prof->ev[i + 1]));
      }
      auto& lp = res.last_profile;
      lp.coarse_ms += ms[0];
      lp.rotate_ms += ms[1];
      lp.scan_ms += ms[2];
      lp.merge_ms += ms[3];
      lp.total_ms += ms[0] + ms[1] + ms[2] + ms[3];
      lp.n_scan_launches += 1;
      if (early_stop) {
        float lead_ms = 0, screen_ms = 0, surv_ms = 0;
        CUVS_HIP_TRY(hipEventElapsedTime(&lead_ms, res.prof->ev[2], res.prof->ev[5]));
        CUVS_HIP_TRY(hipEventElapsedTime(&screen_ms, res.prof->ev[5], res.prof->ev[6]));
        CUVS_HIP_TRY(hipEventElapsedTime(&surv_ms, res.prof->ev[6], res.prof->ev[3]));
        lp.lead_scan_ms += lead_ms;
        lp.screen_ms += screen_ms;
        lp.survivor_scan_ms += surv_ms;
        // which pairs survived: their records are still in the workspace
        uint32_t counts[2] = {0, 0};  // survivors, pairs dropped on their length
        CUVS_HIP_TRY(hipMemcpy(counts, n_survivors, 8, hipMemcpyDeviceToHost));
        const uint32_t n_surv = counts[0];
        lp.n_far_pairs += counts[1];
        std::vector<detail::pair_desc> h_surv(n_surv);
        if (n_surv != 0) {
          CUVS_HIP_TRY(hipMemcpy(h_surv.data(), screen_out, size_t(n_surv) * sizeof(detail::pair_desc),
                                 hipMemcpyDeviceToHost));
        }
        const uint64_t row_bytes = uint64_t(ix.n_chunks) * kIndexGroupVecLen;
        for (const auto& d : h_surv) { lp.survivor_bytes += uint64_t((d.n_rows + 31u) & ~31u) * row_bytes; }
        lp.n_surviving_pairs += n_surv;
        lp.n_screened_pairs += uint64_t(nq) * (P - lead);
      }
    }
  }
  if (prof) {
    std::vector<unsigned long long> slots(size_t(detail::kStatSlots) * 4);
    CUVS_HIP_TRY(hipMemcpyAsync(slots.data(), d_stats, slots.size() * 8, hipMemcpyDeviceToHost, s));
    CUVS_HIP_TRY(hipStreamSynchronize(s));
    unsigned long long h[4] = {0, 0, 0, 0};
    for (size_t i = 0; i < slots.size(); i++) { h[i % 4] += slots[i]; }
    res.last_profile.scan_bytes = h[0];
    res.last_profile.scan_rows  = h[1];
    if (early_stop) {
      res.last_profile.lead_bytes   = h[2];
      // rows x leading bytes the screen reads
      res.last_profile.screen_bytes =
        (h[0] - h[2]) / (uint64_t(ix.n_chunks) * kIndexGroupVecLen) * detail::scan_screen_bytes_per_row(ix.codebook_kind == codebook_gen::PER_CLUSTER, ix.lead_plane.bytes != 0);
    }
  }
  res.reset_workspace();
}
}  // namespace

template <typename T>
struct elem_of;
template <>
struct elem_of<float> {
  static constexpr elem_type value = elem_type::f32;
};
template <>
struct elem_of<_Float16> {
  static constexpr elem_type value = elem_type::f16;
};
template <>
struct elem_of<int8_t> {
  static constexpr elem_type value = elem_type::i8;
};
template <>
struct elem_of<uint8_t> {
  static constexpr elem_type value = elem_type::u8;
};

template <typename T>
void search(cuvs::resources const& res,
            const search_params& params,
            const index<int64_t>& idx,
            device_matrix_view<const T> queries,
            device_matrix_view<int64_t> neighbors,
            device_matrix_view<float> distances,
            const cuvs::neighbors::filtering::base_filter& sample_filter)
{
  // search_with_filtering (ivf_pq_search.cuh:1079-1108)
  CUVS_EXPECTS(
    queries.extent(0) == neighbors.extent(0) && queries.extent(0) == distances.extent(0),
    "Number of rows in output neighbors and distances matrices must equal the number of queries.");
  CUVS_EXPECTS(neighbors.extent(1) == distances.extent(1),
               "Number of columns in output neighbors and distances matrices must equal k");
  search(res, params, idx, queries.data_handle(), elem_of<T>::value, queries.extent(0),
         queries.extent(1), neighbors.data_handle(), distances.data_handle(), neighbors.extent(1),
         sample_filter);
}

#define INSTANTIATE_SEARCH(T)                                                              \
  template void search<T>(cuvs::resources const&, const search_params&, const index<int64_t>&, \
                          device_matrix_view<const T>, device_matrix_view<int64_t>,        \
                          device_matrix_view<float>,                                       \
                          const cuvs::neighbors::filtering::base_filter&);
INSTANTIATE_SEARCH(float)
INSTANTIATE_SEARCH(_Float16)
INSTANTIATE_SEARCH(int8_t)
INSTANTIATE_SEARCH(uint8_t)

}  // namespace cuvs::neighbors::ivf_pq
