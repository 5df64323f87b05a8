/*
 * Table-free code scan for fp32 lookup tables (8-bit codes, L2 metrics, per-subspace codebooks):
 * the LUT + score steps of the reference's compute_similarity kernel
 * (cpp/src/neighbors/ivf_pq/detail/jit_lto_kernels/create_lut_impl.cuh:16-79,
 * compute_score_impl.cuh:55-79) for the launches of an early stop that scan few pairs, the leading
 * and the surviving ones.
 *
 * An fp32 table of 64 subspaces is 64 KB a pair: a CU holds two, and a pair's table is used for a
 * few hundred rows only.  Here nothing is built per pair.  The whole codebook sits in LDS once
 * (pq_dim x 256 entries of pq_len floats: 128 KB for pq_dim 64, pq_len 2), and a lane computes the
 * entry its row's code selects on the spot, with the table builder's own operations (the difference
 * query - centre, minus the codebook component, squared and accumulated by FMA in dimension order),
 * and adds it to its row's fp32 sum in subspace order: the sums are the table kernels' bit for bit.
 *
 * One persistent 1024-thread block per CU; after the codebook is loaded the sixteen waves never
 * meet again.  A wave takes pairs of its own (pair w + i * n_waves): the pair's 2 * 64 differences
 * live in two registers (a lane each) and reach the arithmetic through v_readlane; rows pass in
 * tiles of 64 with the next tile's codes in flight; after every 16 subspaces a tile none of whose
 * rows can still win ends (compute_score's early stop); candidates go to the wave's LDS buffer and
 * are reduced by the wave's radix selection, as in the other wave-per-pair kernel.
 */
#include "scan_wave_select.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr uint32_t kDirectScanThreads = 1024;
constexpr uint32_t kDirectScanMaxK    = 64;
constexpr uint32_t kDirectScanCap     = 128;  // candidate keys a wave buffers: k kept ones and one tile's
constexpr uint32_t kDirectScanCandBase = 256;
constexpr uint32_t kDirectScanBookBase = kDirectScanCandBase + (kDirectScanThreads / 64u) * kDirectScanCap * 8u;

template <int NCH>  // 16-byte chunks a row: pq_dim = 16 * NCH, pq_len 2
__global__ __launch_bounds__(kDirectScanThreads) void scan_direct_kernel(scan_args a)
{
  constexpr uint32_t M   = uint32_t(NCH) * 16u;  // pq_dim
  constexpr uint32_t ROT = M * 2u;
  static_assert(ROT <= 128u, "a pair's differences live in two registers, a lane each");
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = uint32_t(__builtin_amdgcn_readfirstlane(int(tid >> 6)));
  const uint32_t n_pairs =
    uint32_t(__builtin_amdgcn_readfirstlane(int(a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs)));
  constexpr uint32_t WPB = kDirectScanThreads / 64u;
  const uint32_t total   = gridDim.x * WPB;

  // entry (j, c) of the codebook: components t of pq_centers[(j * 2 + t) * 256 + c]
  auto* book = reinterpret_cast<LDS_AS f32x2*>(uintptr_t(kDirectScanBookBase));
  for (uint32_t e = tid; e < M * 256u; e += kDirectScanThreads) {
    f32x2 v;
    v.x     = a.pq_centers[((e >> 8) * 2u + 0u) * 256u + (e & 255u)];
    v.y     = a.pq_centers[((e >> 8) * 2u + 1u) * 256u + (e & 255u)];
    book[e] = v;
  }
  __syncthreads();

  auto* my_cand = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(kDirectScanCandBase)) + wid * kDirectScanCap;

  for (uint32_t p = blockIdx.x * WPB + wid; p < n_pairs; p += total) {
    pair_desc d = a.desc[p];
    {
      // the record is the same in all lanes: say so, and addresses and trip counts stay scalar
      const uint64_t ptr = reinterpret_cast<uint64_t>(d.data);
      const uint32_t hi  = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(ptr >> 32))));
      const uint32_t lo  = uint32_t(__builtin_amdgcn_readfirstlane(int(uint32_t(ptr))));
      d.data             = reinterpret_cast<const uint8_t*>((uint64_t(hi) << 32) | uint64_t(lo));
      d.q                = uint32_t(__builtin_amdgcn_readfirstlane(int(d.q)));
      d.slot             = uint32_t(__builtin_amdgcn_readfirstlane(int(d.slot)));
      d.label            = uint32_t(__builtin_amdgcn_readfirstlane(int(d.label)));
      d.sample_off       = uint32_t(__builtin_amdgcn_readfirstlane(int(d.sample_off)));
      d.n_rows           = uint32_t(__builtin_amdgcn_readfirstlane(int(d.n_rows)));
    }
    const uint32_t n_rows   = d.n_rows;
    unsigned long long* out = a.out_keys + uint64_t(d.slot) * a.k;
    uint32_t wcount         = 0;
    if (n_rows != 0) {
      const uint8_t* list_data = d.data;
      const int64_t* list_ids  = a.filter_bits != nullptr ? a.inds_ptrs[d.label] : nullptr;
      // (rotated query - rotated centre): dimensions 0..63 in dv0, 64..127 in dv1, a lane each
      const float* qp = a.rot_q + uint64_t(d.q) * a.rot_dim;
      const float* cp = a.centers_rot + uint64_t(d.label) * a.rot_dim;
      const float dv0 = lane < ROT ? qp[lane] - cp[lane] : 0.0f;
      const float dv1 = lane + 64u < ROT ? qp[lane + 64u] - cp[lane + 64u] : 0.0f;
      uint32_t thr    = uint32_t(__builtin_amdgcn_readfirstlane(int(a.query_kth[d.q])));
      float thr_f     = thr >= 0xFF800000u ? __uint_as_float(0x7F800000u) : unorder_f32(thr);

      auto load_row = [&](uint32_t row, u32x4 (&dst)[NCH]) {
        const uintptr_t base = reinterpret_cast<uintptr_t>(list_data) + uint64_t(row >> 5) * (uint64_t(NCH) * 512u) +
                               uint64_t(row & 31u) * 16u;
#pragma unroll
        for (int m = 0; m < NCH; m++) { dst[m] = *reinterpret_cast<const GLOBAL_AS u32x4*>(base + uint64_t(m) * 512u); }
      };
      auto take = [&](float score, bool valid, uint32_t row) {
        const unsigned long long mask = __builtin_amdgcn_ballot_w64(valid && score <= thr_f);
        if (mask == 0ull) { return; }
        if (wcount + 64u > kDirectScanCap) {
          // make room (the buffer holds more than k keys): keep the k best and tighten the bound
          const uint32_t t2 = wcount <= 64u ? wave_select_keys<1>(my_cand, lane, wcount, a.k)
                                            : wave_select_keys<2>(my_cand, lane, wcount, a.k);
          wcount = a.k;
          if (t2 < thr) {
            thr   = t2;
            thr_f = unorder_f32(thr);
          }
        }
        const uint32_t okey            = order_f32(score);
        const bool pass                = ((mask >> lane) & 1ull) != 0ull && okey <= thr;
        const unsigned long long mask2 = __builtin_amdgcn_ballot_w64(pass);
        const uint32_t below =
          __builtin_amdgcn_mbcnt_hi(uint32_t(mask2 >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask2), 0u));
        if (pass) { my_cand[wcount + below] = (static_cast<unsigned long long>(okey) << 32) | (d.sample_off + row); }
        wcount += uint32_t(__popcll(mask2));
      };

      const uint32_t n_tiles = (n_rows + 63u) >> 6;
      u32x4 cur[NCH], ahead[NCH];
      load_row(lane < n_rows ? lane : 0u, cur);
      for (uint32_t tile = 0; tile < n_tiles; tile++) {
        const uint32_t row = tile * 64u + lane;
        {
          // the next tile's codes, requested without a condition (past the end: row 0 again)
          const uint32_t nr = row + 64u;
          load_row(nr < n_rows ? nr : 0u, ahead);
        }
        bool valid = row < n_rows;
        if (list_ids != nullptr && valid) {
          const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[row];
          valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
        }
        // sums of an L2 scan are not negative: past the bound means past its bits
        const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
        float acc                = 0.0f;
        bool live                = __builtin_amdgcn_ballot_w64(valid) != 0ull;
#pragma unroll
        for (int m = 0; m < NCH; m++) {
          if (live) {
            const uint32_t w[4] = {cur[m].x, cur[m].y, cur[m].z, cur[m].w};
#pragma unroll
            for (int kk = 0; kk < 16; kk++) {
              constexpr int kDummy = 0;
              (void)kDummy;
              const int j      = m * 16 + kk;
              const uint32_t c = (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu;
              const f32x2 b    = book[j * 256 + int(c)];
              // the pair's differences of dimensions 2 j, 2 j + 1
              const int l0   = (2 * j) & 63;
              const float d0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(j < 32 ? dv0 : dv1), l0));
              const float d1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(j < 32 ? dv0 : dv1), l0 + 1));
              float score    = 0.0f;
              float diff     = d0 - b.x;
              score          = fmaf(diff, diff, score);
              diff           = d1 - b.y;
              score          = fmaf(diff, diff, score);
              acc += score;
            }
            if (m + 1 < NCH) { live = __builtin_amdgcn_ballot_w64(valid && !(__float_as_uint(acc) > stop_bits)) != 0ull; }
          }
        }
        if (acc != acc) { valid = false; }
        if (live) { take(acc, valid, row); }
#pragma unroll
        for (int m = 0; m < NCH; m++) { cur[m] = ahead[m]; }
      }
      if (wcount >= a.k) {
        const uint32_t kth = wcount <= 64u ? wave_select_keys<1>(my_cand, lane, wcount, a.k)
                                           : wave_select_keys<2>(my_cand, lane, wcount, a.k);
        wcount = a.k;
        if (lane == 0) { atomicMin(&a.query_kth[d.q], kth); }
      }
    }
    for (uint32_t t = lane; t < a.k; t += 64u) { out[t] = t < wcount ? my_cand[t] : kInvalidKey; }
  }
}

template <int NCH>
void launch_direct_instance(const scan_args& a, hipStream_t stream)
{
  auto kernel       = scan_direct_kernel<NCH>;
  const size_t smem = kDirectScanBookBase + size_t(NCH) * 16 * 256 * 8;
  static const int attr_set = [&] {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
    return 1;
  }();
  (void)attr_set;
  constexpr uint32_t wpb = kDirectScanThreads / 64u;
  uint32_t grid          = uint32_t(device_cu_count());
  if (a.n_pairs_dev == nullptr) {
    const uint32_t needed = (a.n_pairs + wpb - 1u) / wpb;
    if (grid > needed) { grid = needed; }
    if (grid == 0) { return; }
  }
  kernel<<<grid, kDirectScanThreads, smem, stream>>>(a);
  CUVS_HIP_TRY(hipGetLastError());
}

}  // namespace

bool scan_direct_supported(const scan_args& a)
{
  const bool l2 = a.metric == int(DistanceType::L2Expanded) || a.metric == int(DistanceType::L2SqrtExpanded);
  if (!l2 || !a.fused || a.pq_bits != 8 || a.per_cluster || a.k > kDirectScanMaxK) { return false; }
  if (a.lut_dtype != CUDA_R_32F || a.out_half) { return false; }
  if (a.pq_len != 2 || a.rot_dim != a.pq_dim * a.pq_len) { return false; }
  return a.pq_dim == 64 || a.pq_dim == 48 || a.pq_dim == 32;
}

bool launch_scan_direct(const scan_args& a, hipStream_t stream)
{
  if (!scan_direct_supported(a) || a.n_queries == 0 || a.desc == nullptr) { return false; }
  switch (a.pq_dim) {
    case 64: launch_direct_instance<4>(a, stream); break;
    case 48: launch_direct_instance<3>(a, stream); break;
    default: launch_direct_instance<2>(a, stream); break;
  }
  return true;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
