/*
 * Persistent LUT + code-scan kernel for 8-bit codes (the configurations the benchmark is quoted
 * on).  Same arithmetic as the generic scan kernel in kernels.hip, organised for CDNA4:
 *
 *   - a fixed grid of 256-thread blocks (as many as fit on the chip) pulls (query, probe) pairs
 *     from a global counter, in list order, so that neighbouring blocks stream the same list
 *     while it is hot in L2;
 *   - thread t owns codebook entry t of every subspace and keeps those pq_dim * pq_len floats in
 *     registers for the whole kernel: building a lookup table costs no memory traffic besides
 *     one broadcast LDS read per subspace and one LDS write per entry;
 *   - the list's codes are read with one 16-byte load per 16 codes, the next row is in flight
 *     while the current one is scored, and the first row is requested before the table is built;
 *   - candidates that beat the query's running k-th distance are appended to an LDS buffer with
 *     one wave-aggregated atomic; the block only synchronises to prune the buffer every 1792
 *     rows and at the end of the list.
 */
#include "device_utils.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

constexpr uint32_t kFastCap      = 2048;                // candidate keys held per block
constexpr uint32_t kFastMaxK     = 256;                 // largest k the buffer arithmetic allows
constexpr uint32_t kFastSegIters = (kFastCap - kFastMaxK) / kBlock;  // row iterations per prune

struct fast_tail {
  uint32_t count;
  uint32_t thr;
  uint32_t work;
  uint32_t pad;
};

/** Keep the k smallest keys of cand[0..count) sorted at the front; publish the k-th score.
 *  `cnt` is the candidate count every thread read between two barriers; returns after a barrier.
 *  No-op when cnt < k. */
__device__ __forceinline__ void block_prune(unsigned long long* cand, fast_tail* tail, uint32_t k,
                                            uint32_t cnt)
{
  const uint32_t tid = threadIdx.x;
  if (cnt < k) { return; }
  if (cnt <= 64u) {
    // one wave ranks the candidates by all-pairs comparison (keys are distinct)
    if (tid < 64u) {
      const unsigned long long key = tid < cnt ? cand[tid] : kInvalidKey;
      const uint32_t lo            = uint32_t(key);
      const uint32_t hi            = uint32_t(key >> 32);
      uint32_t rank                = 0;
      for (uint32_t j = 0; j < cnt; j++) {
        const uint32_t olo = __builtin_amdgcn_readlane(lo, j);
        const uint32_t ohi = __builtin_amdgcn_readlane(hi, j);
        const unsigned long long other = (static_cast<unsigned long long>(ohi) << 32) | olo;
        rank += other < key ? 1u : 0u;
      }
      if (tid < cnt && rank < k) { cand[rank] = key; }
      if (tid < cnt && rank == k - 1u) { tail->thr = hi; }
      if (tid == 0) { tail->count = k; }
    }
    __syncthreads();
    return;
  }
  uint32_t n2 = 128;
  while (n2 < cnt) { n2 <<= 1; }
  for (uint32_t t = cnt + tid; t < n2; t += kBlock) { cand[t] = kInvalidKey; }
  __syncthreads();
  block_bitonic_sort(cand, n2);
  if (tid == 0) {
    tail->count = k;
    tail->thr   = uint32_t(cand[k - 1] >> 32);
  }
  __syncthreads();
}

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
__global__ __launch_bounds__(kBlock, 2) void scan_fast_kernel(scan_args a, uint32_t* work_counter)
{
  using traits = lut_traits<LUT>;
  using lut_t  = typename traits::storage;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  constexpr int M              = NCH * 16;  // pq_dim
  constexpr uint32_t lut_bytes = uint32_t(M) * 256u * uint32_t(sizeof(lut_t));
  constexpr uint32_t n_diff    = uint32_t(M) * PQ_LEN * (IP ? 2u : 1u);

  extern __shared__ __align__(16) unsigned char dyn_smem[];
  lut_t* lut               = reinterpret_cast<lut_t*>(dyn_smem);
  float* base_diff         = reinterpret_cast<float*>(dyn_smem + lut_bytes);
  unsigned long long* cand = reinterpret_cast<unsigned long long*>(dyn_smem + lut_bytes + n_diff * 4u);
  fast_tail* tail          = reinterpret_cast<fast_tail*>(cand + kFastCap);

  const uint32_t tid     = threadIdx.x;
  const uint32_t n_pairs = a.n_queries * a.n_probes;

  // codebook entry `tid` of every subspace, resident for the whole kernel
  float book[PER_CLUSTER ? 1 : M][PQ_LEN];
  if (!PER_CLUSTER) {
#pragma unroll
    for (int j = 0; j < M; j++) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) { book[j][t] = a.pq_centers[(j * PQ_LEN + t) * 256 + tid]; }
    }
  }

  for (;;) {
    if (tid == 0) { tail->work = atomicAdd(work_counter, 1u); }
    __syncthreads();  // also: every thread is done with the previous pair's table and candidates
    const uint32_t it = tail->work;
    if (it >= n_pairs) { break; }
    const uint32_t pair       = a.pair_order != nullptr ? a.pair_order[it] : it;
    const uint32_t q          = pair / a.n_probes;
    const uint32_t p          = pair - q * a.n_probes;
    const uint32_t label      = a.probes[uint64_t(q) * a.n_probes + p];
    const uint32_t* chunk_row = a.chunk_indices + uint64_t(q) * a.n_probes;
    const uint32_t sample_off = p > 0 ? chunk_row[p - 1] : 0u;
    const uint32_t n_rows     = chunk_row[p] - sample_off;
    unsigned long long* out   = a.out_keys + (uint64_t(q) * a.n_probes + p) * a.k;
    if (n_rows == 0) {
      for (uint32_t r = tid; r < a.k; r += kBlock) { out[r] = kInvalidKey; }
      continue;
    }

    // request the first row of codes before the table is built
    const uint8_t* list_data = a.data_ptrs[label];
    const int64_t* list_ids  = a.filter_bits != nullptr ? a.inds_ptrs[label] : nullptr;
    uint4 cur[NCH];
    {
      const uint32_t i0 = tid < n_rows ? tid : 0u;
      const uint4* ptr  = reinterpret_cast<const uint4*>(list_data + uint64_t(i0 >> 5) * (NCH * 512u) +
                                                        uint64_t(i0 & 31u) * 16u);
#pragma unroll
      for (int m = 0; m < NCH; m++) { cur[m] = ptr[m * 32]; }
    }

    /* ---- per-dimension query / centre terms ---- */
    const float* rq = a.rot_q + uint64_t(q) * (M * PQ_LEN);
    const float* cr = a.centers_rot + uint64_t(label) * (M * PQ_LEN);
    for (uint32_t i = tid; i < uint32_t(M * PQ_LEN); i += kBlock) {
      if (!IP) {
        base_diff[i] = rq[i] - cr[i];
      } else {
        const float qv       = rq[i];
        base_diff[2 * i]     = qv;
        base_diff[2 * i + 1] = cr[i] * qv;
      }
    }
    float cbook[PQ_LEN];
    if (PER_CLUSTER) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        cbook[t] = a.pq_centers[(uint64_t(label) * PQ_LEN + t) * 256 + tid];
      }
    }
    if (tid == 0) {
      tail->count = 0;
      tail->thr   = 0xFFFFFFFFu;
    }
    __syncthreads();

    /* ---- lookup table ---- */
#pragma unroll
    for (int j = 0; j < M; j++) {
      float score = 0.0f;
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        const float pqc = PER_CLUSTER ? cbook[t] : book[PER_CLUSTER ? 0 : j][t];
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
    __syncthreads();

    /* ---- scan ---- */
    uint32_t thr           = a.query_kth[q];
    const uint32_t n_iters = (n_rows + kBlock - 1u) / kBlock;
    for (uint32_t iter = 0; iter < n_iters; iter++) {
      const uint32_t i = iter * kBlock + tid;
      // next row in flight while this one is scored
      uint4 nxt[NCH];
      {
        const uint32_t in = i + kBlock;
        const uint32_t i1 = in < n_rows ? in : 0u;
        const uint4* ptr  = reinterpret_cast<const uint4*>(
          list_data + uint64_t(i1 >> 5) * (NCH * 512u) + uint64_t(i1 & 31u) * 16u);
#pragma unroll
        for (int m = 0; m < NCH; m++) { nxt[m] = ptr[m * 32]; }
      }
      bool valid = i < n_rows;
      if (valid && list_ids != nullptr) {
        const int64_t id = list_ids[i];
        valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
      }
      acc_t acc = acc_t(0);
#pragma unroll
      for (int m = 0; m < NCH; m++) {
        const uint32_t w[4] = {cur[m].x, cur[m].y, cur[m].z, cur[m].w};
#pragma unroll
        for (int kk = 0; kk < 16; kk++) {
          const uint32_t c = (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu;
          const lut_t e    = lut[(m * 16 + kk) * 256 + c];
          if (OUT_HALF) {
            acc = acc_t(acc + traits::to_half(e));
          } else {
            acc = acc_t(acc + traits::to_float(e));
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
        if (below == 0u && pass) { base = atomicAdd(&tail->count, uint32_t(__popcll(mask))); }
        base = __shfl(base, __ffsll(static_cast<long long>(mask)) - 1, 64);
        if (pass) { cand[base + below] = (static_cast<unsigned long long>(okey) << 32) | (sample_off + i); }
      }
#pragma unroll
      for (int m = 0; m < NCH; m++) { cur[m] = nxt[m]; }
      if ((iter + 1u) % kFastSegIters == 0u && iter + 1u < n_iters) {
        __syncthreads();
        const uint32_t seg_cnt = tail->count;
        __syncthreads();
        block_prune(cand, tail, a.k, seg_cnt);
        const uint32_t t2 = tail->thr;
        thr               = t2 < thr ? t2 : thr;
      }
    }
    __syncthreads();
    const uint32_t before = tail->count;
    __syncthreads();
    block_prune(cand, tail, a.k, before);
    const uint32_t cnt = before < a.k ? before : a.k;
    for (uint32_t r = tid; r < a.k; r += kBlock) { out[r] = r < cnt ? cand[r] : kInvalidKey; }
    if (tid == 0 && before >= a.k) { atomicMin(&a.query_kth[q], tail->thr); }
  }
}

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
void launch_instance(const scan_args& a, uint32_t* work_counter, hipStream_t stream)
{
  using lut_t = typename lut_traits<LUT>::storage;
  auto kernel = scan_fast_kernel<NCH, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP>;
  const size_t smem = size_t(NCH) * 16 * 256 * sizeof(lut_t) + size_t(NCH) * 16 * PQ_LEN * (IP ? 2 : 1) * 4 +
                      size_t(kFastCap) * 8 + sizeof(fast_tail);
  static int blocks_per_cu = 0;  // per instance
  static int n_cu          = 0;
  if (blocks_per_cu == 0) {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
    int occ = 0;
    CUVS_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, kBlock, smem));
    int dev = 0;
    CUVS_HIP_TRY(hipGetDevice(&dev));
    CUVS_HIP_TRY(hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    blocks_per_cu = occ > 0 ? occ : 1;
  }
  const uint32_t n_pairs = a.n_queries * a.n_probes;
  uint32_t grid          = uint32_t(blocks_per_cu) * uint32_t(n_cu);
  if (grid > n_pairs) { grid = n_pairs; }
  launch_fill_u32(work_counter, 0, 1, stream);
  kernel<<<grid, kBlock, smem, stream>>>(a, work_counter);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int NCH, int PQ_LEN, bool PER_CLUSTER>
bool launch_types(const scan_args& a, uint32_t* wc, hipStream_t s)
{
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (!ip) {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_32F) { launch_instance<NCH, PQ_LEN, LUT_F32, false, PER_CLUSTER, false>(a, wc, s); return true; }
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, false>(a, wc, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8U, false, PER_CLUSTER, false>(a, wc, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, false>(a, wc, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8U, true, PER_CLUSTER, false>(a, wc, s); return true; }
    }
  } else {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_32F) { launch_instance<NCH, PQ_LEN, LUT_F32, false, PER_CLUSTER, true>(a, wc, s); return true; }
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, true>(a, wc, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8S, false, PER_CLUSTER, true>(a, wc, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, true>(a, wc, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_instance<NCH, PQ_LEN, LUT_FP8S, true, PER_CLUSTER, true>(a, wc, s); return true; }
    }
  }
  return false;
}

template <int NCH, int PQ_LEN>
bool launch_kind(const scan_args& a, uint32_t* wc, hipStream_t s)
{
  return a.per_cluster ? launch_types<NCH, PQ_LEN, true>(a, wc, s) : launch_types<NCH, PQ_LEN, false>(a, wc, s);
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

bool launch_scan_fast(const scan_args& a, uint32_t* work_counter, hipStream_t stream)
{
  if (!scan_fast_supported(a) || a.n_queries == 0) { return false; }
  if (a.pq_dim == 64 && a.pq_len == 2) { return launch_kind<4, 2>(a, work_counter, stream); }
  if (a.pq_dim == 48 && a.pq_len == 2) { return launch_kind<3, 2>(a, work_counter, stream); }
  if (a.pq_dim == 32 && a.pq_len == 4) { return launch_kind<2, 4>(a, work_counter, stream); }
  return false;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
