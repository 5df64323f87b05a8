/*
 * Persistent LUT + code-scan kernel for 8-bit codes (the configurations the benchmark is quoted
 * on).  Same arithmetic as the generic scan kernel in kernels.hip, organised for CDNA4:
 *
 *   - a fixed grid of 256-thread blocks (as many as fit on the chip) walks the (query, probe)
 *     pairs in list order with a grid-sized stride, so that neighbouring blocks stream the same
 *     list while it is hot in L2; the 32-byte record of a pair is read two pairs ahead and the
 *     pair's first codes, query and centre one pair ahead, so that no dependent global load sits
 *     on the critical path between two pairs;
 *   - thread t owns codebook entry t of every subspace and keeps those pq_dim * pq_len floats in
 *     registers for the whole kernel: building a lookup table costs no memory traffic besides
 *     one broadcast LDS read per subspace and one LDS write per entry;
 *   - the list's codes are read with one 16-byte load per 16 codes, the next row is in flight
 *     while the current one is scored, and the first row is requested before the table is built;
 *   - candidates that beat the query's running k-th distance are appended to an LDS buffer with
 *     one wave-aggregated atomic; the block only synchronises to prune the buffer every 1792
 *     rows and at the end of the list.
 */
#include "scan_block_select.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

/** What a thread fetches ahead of time for the next pair besides its first row of codes. */
template <int PQ_LEN>
struct pair_prefetch {
  float q, c;          // rotated query / rotated centre element `tid`
  float book[PQ_LEN];  // per-cluster codebook entry `tid` (unused for per-subspace codebooks)
  uint32_t thr;        // the query's current k-th score bound
};

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
__global__ __launch_bounds__(kBlock, 2) void scan_fast_kernel(scan_args a)
{
  using traits = lut_traits<LUT>;
  using lut_t  = typename traits::storage;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  constexpr int M              = NCH * 16;  // pq_dim
  constexpr uint32_t ROT       = uint32_t(M) * PQ_LEN;
  constexpr uint32_t lut_bytes = uint32_t(M) * 256u * uint32_t(sizeof(lut_t));
  constexpr uint32_t n_diff    = ROT * (IP ? 2u : 1u);
  static_assert(ROT <= kBlock, "one thread stages one rotated dimension");

  auto* lut       = reinterpret_cast<LDS_AS lut_t*>(uintptr_t(kLdsBase));
  auto* base_diff = reinterpret_cast<LDS_AS float*>(uintptr_t(kLdsBase + lut_bytes));
  auto* cand = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(kLdsBase + lut_bytes + n_diff * 4u));
  auto* tail = reinterpret_cast<LDS_AS fast_tail*>(uintptr_t(kLdsBase + lut_bytes + n_diff * 4u + kFastCap * 8u));
  const float one = opaque_one();

  const uint32_t tid     = threadIdx.x;
  const uint32_t n_pairs = a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs;
  const uint32_t stride  = gridDim.x;
  if (blockIdx.x >= n_pairs) { return; }  // whole block, before any barrier

  // codebook entry `tid` of every subspace, resident for the whole kernel
  float book[PER_CLUSTER ? 1 : M][PQ_LEN];
  if (!PER_CLUSTER) {
#pragma unroll
    for (int j = 0; j < M; j++) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) { book[j][t] = a.pq_centers[(j * PQ_LEN + t) * 256 + tid]; }
    }
  }

  // List pointers come out of memory, so the compiler cannot tell that they are global addresses
  // and would use flat loads; flat loads count against the LDS counter as well and force every
  // wait on an LDS gather to drain the global prefetches too.  Say explicitly that they are global.
  auto load_row = [&](const uint8_t* list_data, uint32_t row, u32x4 (&dst)[NCH]) {
    const auto* ptr = reinterpret_cast<const GLOBAL_AS u32x4*>(
      reinterpret_cast<uintptr_t>(list_data) + uint64_t(row >> 5) * (NCH * 512u) + uint64_t(row & 31u) * 16u);
#pragma unroll
    for (int m = 0; m < NCH; m++) { dst[m] = ptr[m * 32]; }
  };
  // first row of codes plus the small per-pair operands of pair `d`
  auto fetch = [&](const pair_desc& d, u32x4 (&row0)[NCH], pair_prefetch<PQ_LEN>& f) {
    if (d.n_rows != 0) {
      load_row(d.data, tid < d.n_rows ? tid : 0u, row0);
      if (tid < ROT) {
        f.q = a.rot_q[uint64_t(d.q) * ROT + tid];
        f.c = a.centers_rot[uint64_t(d.label) * ROT + tid];
      }
      if (PER_CLUSTER) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          f.book[t] = a.pq_centers[(uint64_t(d.label) * PQ_LEN + t) * 256 + tid];
        }
      }
      f.thr = a.query_kth[d.q];
    }
  };

  // software pipeline over the block's pairs: records two pairs ahead, operands one pair ahead
  uint32_t it     = blockIdx.x;
  pair_desc cur_d = a.desc[it];
  pair_desc nxt_d = a.desc[it + stride < n_pairs ? it + stride : it];
  u32x4 cur[NCH];    // codes of the row being scored
  u32x4 ahead[NCH];  // codes of the next row of this list, or of the first row of the next pair
  pair_prefetch<PQ_LEN> cur_f, nxt_f;
  fetch(cur_d, cur, cur_f);

  for (;;) {
    const bool has_next     = it + stride < n_pairs;
    const uint32_t it_after = it + 2u * stride < n_pairs ? it + 2u * stride : it;
    const pair_desc after_d = a.desc[it_after];

    const uint32_t n_rows     = cur_d.n_rows;
    const uint32_t sample_off = cur_d.sample_off;
    const uint32_t q          = cur_d.q;
    unsigned long long* out   = a.out_keys + uint64_t(cur_d.slot) * a.k;
    if (n_rows == 0) {
      for (uint32_t r = tid; r < a.k; r += kBlock) { out[r] = kInvalidKey; }
      if (has_next) { fetch(nxt_d, ahead, nxt_f); }
    } else {
      const uint8_t* list_data = cur_d.data;
      const int64_t* list_ids  = a.filter_bits != nullptr ? a.inds_ptrs[cur_d.label] : nullptr;

      /* ---- per-dimension query / centre terms ---- */
      if (tid < ROT) {
        if (!IP) {
          base_diff[tid] = cur_f.q - cur_f.c;
        } else {
          base_diff[2 * tid]     = cur_f.q;
          base_diff[2 * tid + 1] = cur_f.c * cur_f.q;
        }
      }
      if (tid == 0) {
        tail->count = 0;
        tail->thr   = 0xFFFFFFFFu;
      }
      lds_barrier();

      /* ---- lookup table ---- */
#pragma unroll
      for (int j = 0; j < M; j++) {
        float score = 0.0f;
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          const float pqc = PER_CLUSTER ? cur_f.book[t] : book[PER_CLUSTER ? 0 : j][t];
          const int d     = j * PQ_LEN + t;
          if (!IP) {
            float diff = base_diff[d];
            diff -= pqc;
            score = fmaf(diff, diff, score);
          } else {
            const float qv = base_diff[2 * d];
            score -= base_diff[2 * d + 1];
            score = fmaf(-qv, pqc, score);
          }
        }
        lut[j * 256 + tid] = traits::encode(score);
      }
      lds_barrier();

      /* ---- scan ---- */
      uint32_t thr           = cur_f.thr;
      const uint32_t n_iters = (n_rows + kBlock - 1u) / kBlock;
      for (uint32_t iter = 0; iter < n_iters; iter++) {
        const uint32_t i = iter * kBlock + tid;
        // keep one row in flight: the next row of this list, or the first row of the next pair
        if (iter + 1u < n_iters) {
          const uint32_t in = i + kBlock;
          load_row(list_data, in < n_rows ? in : 0u, ahead);
        } else if (has_next) {
          fetch(nxt_d, ahead, nxt_f);
        }
        bool valid = i < n_rows;
        if (valid && list_ids != nullptr) {
          const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[i];
          valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
        }
        acc_t acc = acc_t(0);
        // whole waves past the end of the list skip the tile; L2 sums only grow, so a wave whose
        // rows are all above the bound after a chunk skips the rest (compute_score's early stop)
        const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
        bool live                = __ballot(valid) != 0ull;
#pragma unroll
        for (int m = 0; m < NCH; m++) {
          if (live) {
            const uint32_t w[4] = {cur[m].x, cur[m].y, cur[m].z, cur[m].w};
#pragma unroll
            for (int kk = 0; kk < 16; kk++) {
              const uint32_t c = (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu;
              const lut_t v    = lut[(m * 16 + kk) * 256 + c];
              if (OUT_HALF) {
                acc = acc_t(acc + traits::to_half(v));
              } else if (LUT == LUT_F16) {
                acc = acc_t(fmaf(traits::to_float(v), one, float(acc)));
              } else {
                acc = acc_t(acc + traits::to_float(v));
              }
            }
            if (!IP && m + 1 < NCH) {
              live = __ballot(valid && !(__float_as_uint(float(acc)) > stop_bits)) != 0ull;
            }
          }
        }
        if (a.metric == int(DistanceType::CosineExpanded)) { acc = acc_t(acc + acc_t(1)); }
        const float score_f = float(acc);
        if (score_f != score_f) { valid = false; }
        const uint32_t okey = order_f32(score_f);
        const bool pass     = valid && okey <= thr;
        const unsigned long long mask = __ballot(pass);
        if (mask != 0ull) {
          const uint32_t below =
            __builtin_amdgcn_mbcnt_hi(uint32_t(mask >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask), 0u));
          uint32_t base = 0;
          if (below == 0u && pass) {
            base = __hip_atomic_fetch_add(&tail->count, uint32_t(__popcll(mask)), __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_WORKGROUP);
          }
          base = __shfl(base, __ffsll(static_cast<long long>(mask)) - 1, 64);
          if (pass) { cand[base + below] = (static_cast<unsigned long long>(okey) << 32) | (sample_off + i); }
        }
        if (iter + 1u < n_iters) {
#pragma unroll
          for (int m = 0; m < NCH; m++) { cur[m] = ahead[m]; }
          if ((iter + 1u) % kFastSegIters == 0u) {
            lds_barrier();
            const uint32_t seg_cnt = tail->count;
            lds_barrier();
            block_prune(cand, tail, a.k, seg_cnt);
            const uint32_t t2 = tail->thr;
            thr               = t2 < thr ? t2 : thr;
          }
        }
      }
      lds_barrier();
      const uint32_t before = tail->count;
      lds_barrier();
      block_prune(cand, tail, a.k, before);
      const uint32_t cnt = before < a.k ? before : a.k;
      for (uint32_t r = tid; r < a.k; r += kBlock) { out[r] = r < cnt ? cand[r] : kInvalidKey; }
      if (tid == 0 && before >= a.k) { atomicMin(&a.query_kth[q], tail->thr); }
    }
    if (!has_next) { break; }
    it += stride;
    cur_d = nxt_d;
    nxt_d = after_d;
    cur_f = nxt_f;
#pragma unroll
    for (int m = 0; m < NCH; m++) { cur[m] = ahead[m]; }
  }
}

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
void launch_instance(const scan_args& a, hipStream_t stream)
{
  using lut_t = typename lut_traits<LUT>::storage;
  auto kernel = scan_fast_kernel<NCH, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP>;
  const size_t smem = kLdsBase + size_t(NCH) * 16 * 256 * sizeof(lut_t) +
                      size_t(NCH) * 16 * PQ_LEN * (IP ? 2 : 1) * 4 + size_t(kFastCap) * 8 + sizeof(fast_tail);
  static const int blocks_per_cu = prepare_persistent_kernel(kernel, kBlock, smem, smem);  // per instance
  const int n_cu                 = device_cu_count();
  uint32_t grid = uint32_t(blocks_per_cu) * uint32_t(n_cu);
  if (a.n_pairs_dev == nullptr) {
    if (grid > a.n_pairs) { grid = a.n_pairs; }
    if (grid == 0) { return; }
  }
  kernel<<<grid, kBlock, smem, stream>>>(a);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int NCH, int PQ_LEN, bool PER_CLUSTER>
bool launch_types(const scan_args& a, hipStream_t s)
{
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (!ip) {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_32F) { launch_instance<NCH, PQ_LEN, LUT_F32, false, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8U, false, PER_CLUSTER, false>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8U, true, PER_CLUSTER, false>(a, s); return true; }
    }
  } else {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_32F) { launch_instance<NCH, PQ_LEN, LUT_F32, false, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8S, false, PER_CLUSTER, true>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8S, true, PER_CLUSTER, true>(a, s); return true; }
    }
  }
  return false;
}

template <int NCH, int PQ_LEN>
bool launch_kind(const scan_args& a, hipStream_t s)
{
  return a.per_cluster ? launch_types<NCH, PQ_LEN, true>(a, s) : launch_types<NCH, PQ_LEN, false>(a, s);
}

}  // namespace

bool scan_fast_supported(const scan_args& a)
{
  if (!a.fused || a.pq_bits != 8 || a.k > kFastMaxK) { return false; }
  if (a.rot_dim != a.pq_dim * a.pq_len) { return false; }
  const bool shape = (a.pq_dim == 64 && a.pq_len == 2) || (a.pq_dim == 48 && a.pq_len == 2) ||
                     (a.pq_dim == 32 && a.pq_len == 4);
  return shape;
}

bool launch_scan_fast(const scan_args& a, hipStream_t stream)
{
  if (!scan_fast_supported(a) || a.n_queries == 0 || a.desc == nullptr) { return false; }
  if (a.pq_dim == 64 && a.pq_len == 2) { return launch_kind<4, 2>(a, stream); }
  if (a.pq_dim == 48 && a.pq_len == 2) { return launch_kind<3, 2>(a, stream); }
  if (a.pq_dim == 32 && a.pq_len == 4) { return launch_kind<2, 4>(a, stream); }
  return false;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
