/*
 * Pairs that cannot matter, told apart without touching a row (L2 metrics).
 *
 * A row's score is, in exact arithmetic, |r - b|^2 for the pair's residual r = rotated query -
 * rotated centre and the row's decoded residual b, so it is at least (|r| - |b|)^2, and |b| is at
 * most the list's radius (list_radius_kernel, kept with the index).  |r|^2 needs no pass over the
 * pair's dimensions either: the probe selection has q . c for every probed list already (its
 * fp32 score is |c|^2 - 2 q . c with the stored |c|^2), and
 *
 *   |r|^2 = |R q|^2 + |c_rot|^2 - 2 (R q) . c_rot,   (R q) . c_rot = q . (R^T c_rot),
 *
 * where R^T c_rot equals the stored centre c up to a vector whose length e the index measures per
 * list (zero for a rotation with orthonormal columns and centres rotated by it; whatever the
 * model's tensors hold otherwise).  So |r|^2 >= |R q|^2 + |c_rot|^2 - (|c|^2 - score) - 2 |q| e
 * minus a rounding allowance, from two numbers per query, four per list and the probe's score.
 * The screened pairs whose bound lies past their query's k-th best so far are left out of the
 * record list the screening kernel walks; the others keep their order (the lists' order).
 *
 * Inner product: a row's score is -(R q) . c_rot - (R q) . b, at least
 * -(R q) . c_rot - |R q| radius, and -(R q) . c_rot is the probe selection's score (-q . c) up to
 * |q| e.  What the computed sum can lose against that is relative to the magnitudes of the table's
 * entries, whose sum over the subspaces is at most |R q| (|c_rot| + radius).  Cosine: the scan's
 * query is R q / |R q|, so the probe selection's score (of the query as it came) is divided by
 * |R q| first, and the scans add 1 to a row's sum.
 */
#include "device_utils.cuh"

#include <cmath>
#include <cstddef>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kTermThreads = 256;

/** One block per list: the stored squared norm, |c_rot|^2 and e = |R^T c_rot - c| (rounded up). */
__global__ __launch_bounds__(kTermThreads) void center_terms_kernel(
  const float* __restrict__ centers, const float* __restrict__ centers_rot, const float* __restrict__ rotation,
  uint32_t dim, uint32_t dim_ext, uint32_t rot_dim, int identity, float4* __restrict__ terms)
{
  __shared__ float sums[2][kTermThreads / 64];
  const uint32_t l   = blockIdx.x;
  const uint32_t tid = threadIdx.x;
  const float* c     = centers + uint64_t(l) * dim_ext;
  const float* cr    = centers_rot + uint64_t(l) * rot_dim;
  float n2 = 0.0f, e2 = 0.0f;
  for (uint32_t k = tid; k < rot_dim; k += kTermThreads) { n2 = fmaf(cr[k], cr[k], n2); }
  for (uint32_t d = tid; d < dim; d += kTermThreads) {
    float back = 0.0f;  // (R^T c_rot)[d]; rotation is [rot_dim, dim]
    if (identity) {
      back = cr[d];
    } else {
      for (uint32_t k = 0; k < rot_dim; k++) { back = fmaf(rotation[uint64_t(k) * dim + d], cr[k], back); }
    }
    const float t = back - c[d];
    e2            = fmaf(t, t, e2);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    n2 += __shfl_xor(n2, off, 64);
    e2 += __shfl_xor(e2, off, 64);
  }
  if ((tid & 63u) == 0) {
    sums[0][tid >> 6] = n2;
    sums[1][tid >> 6] = e2;
  }
  __syncthreads();
  if (tid == 0) {
    for (uint32_t w = 1; w < kTermThreads / 64; w++) {
      n2 += sums[0][w];
      e2 += sums[1][w];
    }
    // e also covers what the sums above may have lost: 1e-5 of the centre's length
    const float e = sqrtf(e2) * (1.0f + 1e-5f) + 1e-5f * sqrtf(n2);
    terms[l]      = make_float4(c[dim], n2, e, 0.0f);
  }
}

/** One wave per query: |rot_q|^2 (inner product: 1; cosine: 1 / |R q|, what the scan's query was
 *  divided by), |q| (rounded up), the query's bound as a number, |rot_q| (rounded up). */
__global__ __launch_bounds__(256) void far_query_terms_kernel(const float* __restrict__ rot_q,
                                                              const float* __restrict__ qf, uint32_t rot_dim,
                                                              uint32_t dim, const uint32_t* __restrict__ query_kth,
                                                              uint32_t n_queries, int ip,
                                                              const float* __restrict__ rotation_t, int identity,
                                                              float4* __restrict__ qterms)
{
  const uint32_t q    = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63u;
  if (q >= n_queries) { return; }
  float a = 0.0f, n = 0.0f;
  for (uint32_t k = lane; k < rot_dim; k += 64u) {
    const float v = rot_q[uint64_t(q) * rot_dim + k];
    a             = fmaf(v, v, a);
  }
  for (uint32_t d = lane; d < dim; d += 64u) {
    const float v = qf[uint64_t(q) * dim + d];
    n             = fmaf(v, v, n);
  }
  float rq = 0.0f;  // cosine: |R q|^2 of the query before it was normalised
  if (ip == 2 && !identity) {
    for (uint32_t k = lane; k < rot_dim; k += 64u) {
      float y = 0.0f;
      for (uint32_t d = 0; d < dim; d++) { y = fmaf(rotation_t[uint64_t(d) * rot_dim + k], qf[uint64_t(q) * dim + d], y); }
      rq = fmaf(y, y, rq);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    a += __shfl_xor(a, off, 64);
    n += __shfl_xor(n, off, 64);
    rq += __shfl_xor(rq, off, 64);
  }
  if (lane == 0) {
    if (ip == 1) { a = 1.0f; }
    if (ip == 2) { a = 1.0f / sqrtf(identity ? n : rq); }
    const uint32_t thr = query_kth[q];
    // ordered score words: non-negative numbers have the top bit set; no bound yet reads as a NaN.
    // (L2 scores are not negative: a word below that range bounds them at zero, as in the scans.)
    const float bound = ip ? unorder_f32(thr) : __uint_as_float(thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u);
    float len = 0.0f;  // |rot_q|
    if (ip != 0) {
      float l2 = 0.0f;
      for (uint32_t k = 0; k < rot_dim; k++) { l2 = fmaf(rot_q[uint64_t(q) * rot_dim + k], rot_q[uint64_t(q) * rot_dim + k], l2); }
      len = sqrtf(l2);
    } else {
      len = sqrtf(a);
    }
    qterms[q] = make_float4(a, sqrtf(n) * (1.0f + 1e-5f), bound, len * (1.0f + 1e-5f));
  }
}

/** Is every row of the pair's list provably past the query's bound? */
__device__ __forceinline__ bool pair_is_far(const far_args& f, uint32_t q, uint32_t slot, uint32_t label)
{
  const float4 qt = f.qterms[q];
  const float4 ct = f.center_terms[label];
  // (the score by slot and the query's flag are requested together: the flag is rarely set)
  float score;
  if (f.probe_scores != nullptr) {
    const uint8_t rows = f.from_rows != nullptr ? f.from_rows[q] : uint8_t(0);
    score              = f.probe_scores[slot];
    if (rows != 0) { score = f.score_rows[uint64_t(q) * f.n_lists + label]; }
  } else {
    score = f.score_rows[uint64_t(q) * f.n_lists + label];
  }
  if (f.ip) {
    const float radius = f.list_radius[label];
    const float c_len  = sqrtf(ct.y) * (1.0f + 1e-6f);
    const float mag    = qt.w * (c_len + radius);  // the entries' magnitudes, summed, at most
    const float sc     = qt.x;                      // 1, or 1 / |R q| (cosine)
    const float lb     = score * sc - qt.y * ct.z * sc - qt.w * radius -
                     (f.eps_rel + 2e-5f) * sc * (fabsf(score) + qt.y * (c_len + ct.z)) - f.tol * mag;
    // cosine: the scans add 1 to a row's sum, in the sums' type (`slack` covers that addition)
    const float lbv = f.ip == 2 ? 1.0f + lb - f.slack : lb;
    return mag < 6.0e4f && lbv > qt.z;  // (a NaN anywhere fails the comparison)
  }
  const float two_dot = ct.x - score;  // 2 q . c
  const float mass    = qt.x + ct.y + fabsf(ct.x) + fabsf(score) + qt.y * qt.y;
  const float r2      = qt.x + ct.y - two_dot - 2.0f * qt.y * ct.z - f.eps_rel * mass;
  if (!(r2 > 0.0f)) { return false; }  // also a NaN anywhere
  const float gap = sqrtf(r2) * (1.0f - 1e-6f) - f.list_radius[label];
  return gap > 0.0f && fminf(gap * gap * f.keep - f.slack, f.cap) > qt.z;
}

constexpr uint32_t kFarThreads = 256;
constexpr uint32_t kFarAhead   = 4;  // records a thread has in flight: every one is a chain of dependent loads
constexpr uint32_t kFarRound   = kFarThreads * kFarAhead;

/** Kept pairs of every block's contiguous run of records. */
__global__ __launch_bounds__(kFarThreads) void far_count_kernel(far_args f)
{
  __shared__ uint32_t wave_counts[kFarThreads / 64];
  const uint32_t tid = threadIdx.x;
  const uint32_t per = (f.n_pairs + gridDim.x - 1u) / gridDim.x;
  const uint32_t i0  = blockIdx.x * per;
  const uint32_t i1  = i0 + per < f.n_pairs ? i0 + per : f.n_pairs;
  uint32_t kept      = 0;
  for (uint32_t s = i0; s < i1; s += kFarRound) {
    uint32_t q[kFarAhead], slot[kFarAhead], label[kFarAhead];
#pragma unroll
    for (uint32_t u = 0; u < kFarAhead; u++) {
      const uint32_t i   = s + u * kFarThreads + tid;
      const pair_desc* d = f.desc + (i < i1 ? i : i1 - 1u);
      q[u]               = d->q;
      slot[u]            = d->slot;
      label[u]           = d->label;
    }
#pragma unroll
    for (uint32_t u = 0; u < kFarAhead; u++) {
      const bool far = pair_is_far(f, q[u], slot[u], label[u]);
      kept += (s + u * kFarThreads + tid < i1 && !far) ? 1u : 0u;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) { kept += __shfl_xor(kept, off, 64); }
  if ((tid & 63u) == 0) { wave_counts[tid >> 6] = kept; }
  __syncthreads();
  if (tid == 0) {
    for (uint32_t w = 1; w < kFarThreads / 64; w++) { kept += wave_counts[w]; }
    f.words[kFarTable + blockIdx.x] = kept;
  }
}

/** The kept records, in their order, behind those of the blocks before.  CLAIM: no counting pass
 *  went before; a block claims the places of every round's kept records with one atomic add on the
 *  count (zero before the launch), so the blocks' runs follow each other in no particular order
 *  (for a list that is put in order of length next anyway). */
template <bool CLAIM>
__global__ __launch_bounds__(kFarThreads) void far_move_kernel(far_args f)
{
  __shared__ uint32_t wave_counts[kFarAhead][kFarThreads / 64];
  __shared__ uint32_t s_base, s_total;
  const uint32_t tid = threadIdx.x, lane = tid & 63u, wid = tid >> 6;
  if (!CLAIM && wid == 0) {
    // blocks before this one, and all of them (the grid has at most kFarBlocks blocks)
    uint32_t before = 0, total = 0;
    for (uint32_t b = lane; b < gridDim.x; b += 64u) {
      const uint32_t c = f.words[kFarTable + b];
      total += c;
      before += b < blockIdx.x ? c : 0u;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      before += __shfl_xor(before, off, 64);
      total += __shfl_xor(total, off, 64);
    }
    if (lane == 0) {
      s_base  = before;
      s_total = total;
    }
  }
  __syncthreads();
  uint32_t base = CLAIM ? 0u : s_base;
  if (!CLAIM && blockIdx.x == 0 && tid == 0) {
    f.words[f.count_word] = s_total;
    atomicAdd(f.words + kFarPairsWord, f.n_pairs - s_total);
  }
  const uint32_t per = (f.n_pairs + gridDim.x - 1u) / gridDim.x;
  const uint32_t i0  = blockIdx.x * per;
  const uint32_t i1  = i0 + per < f.n_pairs ? i0 + per : f.n_pairs;
  for (uint32_t s = i0; s < i1; s += kFarRound) {  // uniform trip count
    u32x4 lo[kFarAhead], hi[kFarAhead];
    bool keep[kFarAhead];
#pragma unroll
    for (uint32_t u = 0; u < kFarAhead; u++) {
      const uint32_t i = s + u * kFarThreads + tid;
      const u32x4* src = reinterpret_cast<const u32x4*>(f.desc + (i < i1 ? i : i1 - 1u));
      lo[u]            = src[0];
      hi[u]            = src[1];
    }
#pragma unroll
    for (uint32_t u = 0; u < kFarAhead; u++) {
      const bool far = pair_is_far(f, lo[u].z, lo[u].w, hi[u].x);  // q, slot, label
      keep[u]        = s + u * kFarThreads + tid < i1 && !far;
    }
    unsigned long long votes[kFarAhead];
#pragma unroll
    for (uint32_t u = 0; u < kFarAhead; u++) {
      votes[u] = __builtin_amdgcn_ballot_w64(keep[u]);
      if (lane == 0) { wave_counts[u][wid] = uint32_t(__popcll(votes[u])); }
    }
    __syncthreads();
    if constexpr (CLAIM) {
      if (tid == 0) {
        uint32_t all = 0;
#pragma unroll
        for (uint32_t u = 0; u < kFarAhead; u++) {
#pragma unroll
          for (uint32_t w = 0; w < kFarThreads / 64; w++) { all += wave_counts[u][w]; }
        }
        const uint32_t in_round = (i1 - s < kFarRound ? i1 - s : kFarRound);
        s_base = atomicAdd(f.words + f.count_word, all);
        if (in_round != all) { atomicAdd(f.words + kFarPairsWord, in_round - all); }
      }
      __syncthreads();
      base = s_base;
    }
    // records in index order: part u of the round, then wave, then lane
    uint32_t before = 0;
#pragma unroll
    for (uint32_t u = 0; u < kFarAhead; u++) {
      uint32_t pos = base + before + uint32_t(__popcll(votes[u] & ((1ull << lane) - 1ull)));
#pragma unroll
      for (uint32_t w = 0; w < kFarThreads / 64; w++) {
        pos += w < wid ? wave_counts[u][w] : 0u;
        before += wave_counts[u][w];
      }
      if (keep[u]) {
        u32x4* dst = reinterpret_cast<u32x4*>(f.kept + pos);
        dst[0]     = lo[u];
        dst[1]     = hi[u];
        if (f.alive != nullptr) { f.alive[lo[u].w] = 1; }  // by slot
      }
    }
    base += before;
    __syncthreads();  // the counts are read before the next round writes them
  }
}

}  // namespace

void launch_center_terms(const float* centers, const float* centers_rot, const float* rotation, uint32_t n_lists,
                         uint32_t dim, uint32_t dim_ext, uint32_t rot_dim, bool identity, float4* terms,
                         hipStream_t stream)
{
  if (n_lists == 0) { return; }
  center_terms_kernel<<<n_lists, kTermThreads, 0, stream>>>(centers, centers_rot, rotation, dim, dim_ext, rot_dim,
                                                            identity ? 1 : 0, terms);
  CUVS_HIP_TRY(hipGetLastError());
}

void launch_far_filter(const far_args& f, const float* rot_q, const float* qf, uint32_t rot_dim, uint32_t dim,
                       const uint32_t* query_kth, uint32_t n_queries, const float* rotation_t, bool identity,
                       hipStream_t stream)
{
  static_assert(offsetof(pair_desc, q) == 8 && offsetof(pair_desc, slot) == 12 && offsetof(pair_desc, label) == 16,
                "record layout");
  if (n_queries == 0) { return; }
  far_query_terms_kernel<<<(n_queries + 3u) / 4u, 256, 0, stream>>>(rot_q, qf, rot_dim, dim, query_kth, n_queries,
                                                                     f.ip, rotation_t, identity ? 1 : 0, f.qterms);
  CUVS_HIP_TRY(hipGetLastError());
  uint32_t grid = (f.n_pairs + 4u * kFarThreads - 1u) / (4u * kFarThreads);
  grid          = grid < 1u ? 1u : (grid > kFarBlocks ? kFarBlocks : grid);
  if (f.unordered) {
    far_move_kernel<true><<<grid, kFarThreads, 0, stream>>>(f);
    CUVS_HIP_TRY(hipGetLastError());
    return;
  }
  far_count_kernel<<<grid, kFarThreads, 0, stream>>>(f);
  CUVS_HIP_TRY(hipGetLastError());
  far_move_kernel<false><<<grid, kFarThreads, 0, stream>>>(f);
  CUVS_HIP_TRY(hipGetLastError());
}

}  // namespace cuvs::neighbors::ivf_pq::detail
