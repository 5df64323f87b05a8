/*
 * CU-wide LUT + code-scan kernel for 8-bit codes and k <= 64: the variant the benchmark
 * configurations run on.  Same arithmetic as the other scan kernels; the organisation is chosen
 * for occupancy on CDNA4:
 *
 *   - one persistent block of 1024 threads (16 waves) per CU works on G = 4 (query, probe) pairs
 *     at a time, taken in list order (neighbouring pairs usually probe the same list, so the four
 *     wave groups stream the same codes out of L1/L2);
 *   - the per-subspace codebook is spread over the block: thread (c, s) keeps entry c of the
 *     subspaces of quarter s in registers (pq_dim * pq_len / 4 floats), which leaves the register
 *     budget of four waves per SIMD and gives the LDS gathers enough independent work in flight;
 *   - the four lookup tables of an iteration live in LDS side by side (4 x 32 KB for fp16);
 *     all 16 waves build them together, then wave group g scans the list of pair g;
 *   - every wave keeps its own candidate buffer and k-th bound, so the scan needs no barrier; a
 *     wave writes its <= k best candidates of the pair and the per-query merge kernel sees
 *     waves_per_group * k keys per pair;
 *   - two block barriers per iteration; records, query / centre elements and the first tile of
 *     codes of the next iteration are requested one iteration ahead.
 */
#include "device_utils.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

#define LDS_AS __attribute__((address_space(3)))
#define GLOBAL_AS __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte chunk of codes

constexpr uint32_t kQuadThreads = 1024;
constexpr uint32_t kQuadWaves   = kQuadThreads / 64;
constexpr uint32_t kQuadLdsBase = 16;   // see scan_fast.hip: no pointer constant may be null
constexpr uint32_t kQuadMaxK    = 128;

/** Candidate keys a wave buffers: room for k kept ones plus one tile of 64 new ones. */
inline __host__ __device__ uint32_t quad_wave_cap(uint32_t k) { return k <= 64u ? 128u : 192u; }

__device__ __forceinline__ void lds_barrier_q()
{
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

__device__ __forceinline__ float opaque_one_q()
{
  float one = 1.0f;
  asm volatile("" : "+v"(one));
  return one;
}

/** Ascending sort of the first `cap` keys (at most 256) of one wave's buffer: a bitonic network made of
 *  ascending comparators only (each merge starts with a mirror step), run on the next power of two
 *  with the missing top slots standing for keys larger than any other - a comparator that would
 *  touch one of them never swaps, so it is skipped.  Every slot takes part in one comparator per
 *  step, so the two comparators a lane owns in the 256-wide network do not interfere; LDS
 *  operations of a wave execute in program order, so no barrier is needed. */
__device__ __forceinline__ void wave_sort_cap(LDS_AS unsigned long long* buf, uint32_t lane, uint32_t cap)
{
  // comparators per step: half the next power of two
  const uint32_t n_half = cap <= 2u ? 1u : (1u << (31 - __builtin_clz(cap - 1u)));
  auto compare_exchange = [&](uint32_t i, uint32_t l) __attribute__((always_inline)) {
    if (l < cap) {
      const unsigned long long x = buf[i];
      const unsigned long long y = buf[l];
      if (x > y) {
        buf[i] = y;
        buf[l] = x;
      }
    }
  };
#pragma unroll 1
  for (uint32_t size = 2; size <= 2u * n_half; size <<= 1) {
    const uint32_t half = size >> 1;
    for (uint32_t c = lane; c < n_half; c += 64u) {
      const uint32_t base = (c / half) * size;
      const uint32_t off  = c & (half - 1u);
      compare_exchange(base + off, base + size - 1u - off);
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll 1
    for (uint32_t stride = size >> 2; stride > 0; stride >>= 1) {
      for (uint32_t c = lane; c < n_half; c += 64u) {
        const uint32_t i = (c / stride) * (2u * stride) + (c & (stride - 1u));
        compare_exchange(i, i + stride);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
}

template <int PQ_LEN>
struct quad_prefetch {
  float q, c;          // rotated query / centre element for (pair tid / ROT, dimension tid % ROT)
  float book[PQ_LEN];  // per-cluster codebook entries (unused for per-subspace codebooks)
};

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP, int G>
__global__ __launch_bounds__(kQuadThreads, 4) void scan_quad_kernel(scan_args a)
{
  using traits = lut_traits<LUT>;
  using lut_t  = typename traits::storage;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  constexpr int M                = NCH * 16;                   // pq_dim
  constexpr int QUARTER          = M / 4;                      // subspaces whose codebook a thread holds
  constexpr uint32_t ROT         = uint32_t(M) * PQ_LEN;
  constexpr uint32_t WG          = kQuadWaves / G;             // waves per pair
  constexpr uint32_t lut_entries = uint32_t(M) * 256u;
  constexpr uint32_t lut_bytes   = lut_entries * uint32_t(sizeof(lut_t));
  constexpr uint32_t n_diff      = ROT * (IP ? 2u : 1u);
  static_assert(M % 4 == 0, "pq_dim must split into four quarters");
  static_assert(ROT * G <= kQuadThreads, "one thread stages one (pair, dimension)");

  // LDS: G tables | G x staged query/centre terms | per-wave candidate buffers
  constexpr uint32_t off_diff = kQuadLdsBase + uint32_t(G) * lut_bytes;
  constexpr uint32_t off_cand = off_diff + uint32_t(G) * n_diff * 4u;
  auto* lut_all  = reinterpret_cast<LDS_AS lut_t*>(uintptr_t(kQuadLdsBase));
  auto* diff_all = reinterpret_cast<LDS_AS float*>(uintptr_t(off_diff));
  auto* cand_all = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(off_cand));
  const float one = opaque_one_q();

  const uint32_t tid     = threadIdx.x;
  const uint32_t lane    = tid & 63u;
  const uint32_t wid     = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it scalar
  const uint32_t grp     = wid / WG;         // which pair of the iteration this wave scans
  const uint32_t wig     = wid - grp * WG;   // wave index inside its group
  const uint32_t code    = tid & 255u;       // codebook entry this thread builds
  const uint32_t quarter = wid >> 2;         // which quarter of the subspaces
  const uint32_t n_pairs = a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs;
  const uint32_t n_quads = (n_pairs + G - 1u) / G;
  const uint32_t stride  = gridDim.x;
  if (blockIdx.x >= n_quads) { return; }  // whole block, before any barrier
  const uint32_t wave_cap = quad_wave_cap(a.k);
  auto* my_cand          = cand_all + wid * wave_cap;
  auto* my_lut           = lut_all + grp * lut_entries;

  float book[PER_CLUSTER ? 1 : QUARTER][PQ_LEN];
  if (!PER_CLUSTER) {
#pragma unroll
    for (int jj = 0; jj < QUARTER; jj++) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        book[jj][t] = a.pq_centers[((quarter * QUARTER + jj) * PQ_LEN + t) * 256 + code];
      }
    }
  }

  auto load_tile = [&](const uint8_t* list_data, uint32_t row, u32x4 (&dst)[NCH]) {
    const auto* ptr = reinterpret_cast<const GLOBAL_AS u32x4*>(
      reinterpret_cast<uintptr_t>(list_data) + uint64_t(row >> 5) * (NCH * 512u) + uint64_t(row & 31u) * 16u);
#pragma unroll
    for (int m = 0; m < NCH; m++) { dst[m] = ptr[m * 32]; }
  };
  // pair record of slot (quad, g); slots past the end read as an empty pair
  auto record = [&](uint32_t quad, uint32_t g) -> pair_desc {
    const uint32_t slot = quad * G + g;
    pair_desc d         = a.desc[slot < n_pairs ? slot : n_pairs - 1u];
    if (slot >= n_pairs) { d.n_rows = 0; d.slot = 0xFFFFFFFFu; }
    return d;
  };
  // operands of the next iteration: staging element (tid / ROT, tid % ROT), codebook for per-cluster
  auto fetch_small = [&](uint32_t quad, quad_prefetch<PQ_LEN>& f) {
    if (tid < ROT * G) {
      const pair_desc d = record(quad, tid / ROT);
      f.q = 0.0f;
      f.c = 0.0f;
      if (d.n_rows != 0) {
        f.q = a.rot_q[uint64_t(d.q) * ROT + tid % ROT];
        f.c = a.centers_rot[uint64_t(d.label) * ROT + tid % ROT];
      }
    }
  };

  uint32_t quad = blockIdx.x;
  quad_prefetch<PQ_LEN> nxt_f;
  fetch_small(quad, nxt_f);
  pair_desc my_d = record(quad, grp);  // the pair this wave scans in the current iteration
  u32x4 cur[NCH], ahead[NCH];
  if (my_d.n_rows != 0) {
    const uint32_t r0 = wig * 64u + lane;
    load_tile(my_d.data, r0 < my_d.n_rows ? r0 : 0u, cur);
  }
  uint32_t pre_thr = my_d.n_rows != 0 ? a.query_kth[my_d.q] : 0xFFFFFFFFu;

  // stage the first iteration's query / centre terms
  if (tid < ROT * G) {
    auto* dst = diff_all + (tid / ROT) * n_diff;
    if (!IP) {
      dst[tid % ROT] = nxt_f.q - nxt_f.c;
    } else {
      dst[2 * (tid % ROT)]     = nxt_f.q;
      dst[2 * (tid % ROT) + 1] = nxt_f.c * nxt_f.q;
    }
  }
  lds_barrier_q();

  for (;;) {
    const bool has_next     = quad + stride < n_quads;
    const uint32_t nxt_quad = has_next ? quad + stride : quad;
    if (has_next) { fetch_small(nxt_quad, nxt_f); }
    const pair_desc nxt_d = record(nxt_quad, grp);

    /* ---- G lookup tables, built by all waves ---- */
#pragma unroll
    for (int g = 0; g < G; g++) {
      const pair_desc dg = record(quad, g);
      if (dg.n_rows == 0) { continue; }  // uniform
      float cb[PQ_LEN];
      if (PER_CLUSTER) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          cb[t] = a.pq_centers[(uint64_t(dg.label) * PQ_LEN + t) * 256 + code];
        }
      }
      const auto* diff = diff_all + g * n_diff;
      auto* lut        = lut_all + g * lut_entries;
#pragma unroll
      for (int jj = 0; jj < QUARTER; jj++) {
        const uint32_t j = quarter * QUARTER + jj;
        float score      = 0.0f;
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          const float pqc  = PER_CLUSTER ? cb[t] : book[PER_CLUSTER ? 0 : jj][t];
          const uint32_t d = j * PQ_LEN + t;
          if (!IP) {
            float df = diff[d];
            df -= pqc;
            score = fmaf(df, df, score);
          } else {
            const float qv = diff[2 * d];
            score -= diff[2 * d + 1];
            score = fmaf(-qv, pqc, score);
          }
        }
        lut[j * 256 + code] = traits::encode(score);
      }
    }
    lds_barrier_q();  // tables complete; the staged terms are free again

    // stage the next iteration's terms now (read after the barrier that ends this iteration)
    if (has_next && tid < ROT * G) {
      auto* dst = diff_all + (tid / ROT) * n_diff;
      if (!IP) {
        dst[tid % ROT] = nxt_f.q - nxt_f.c;
      } else {
        dst[2 * (tid % ROT)]     = nxt_f.q;
        dst[2 * (tid % ROT) + 1] = nxt_f.c * nxt_f.q;
      }
    }

    /* ---- scan: wave `wig` of group `grp` takes tiles wig, wig + WG, ... of its pair ---- */
    if (my_d.slot != 0xFFFFFFFFu) {
      const uint32_t n_rows     = my_d.n_rows;
      const uint32_t sample_off = my_d.sample_off;
      const uint8_t* list_data  = my_d.data;
      const int64_t* list_ids   = a.filter_bits != nullptr && n_rows != 0 ? a.inds_ptrs[my_d.label] : nullptr;
      const uint32_t n_tiles    = (n_rows + 63u) >> 6;
      uint32_t thr              = pre_thr;
      uint32_t wcount           = 0;
      for (uint32_t tile = wig; tile < n_tiles; tile += WG) {
        const uint32_t i = tile * 64u + lane;
        if (tile + WG < n_tiles) {
          const uint32_t in = i + WG * 64u;
          load_tile(list_data, in < n_rows ? in : 0u, ahead);
        }
        bool valid = i < n_rows;
        if (valid && list_ids != nullptr) {
          const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[i];
          valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
        }
        acc_t acc = acc_t(0);
        // L2 sums only grow: once every row of the tile is past the bound the remaining chunks
        // cannot bring any of them back (early stop of compute_score in the reference)
        const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
        bool live                = true;
#pragma unroll
        for (int m = 0; m < NCH; m++) {
          if (live) {
            const uint32_t w[4] = {cur[m].x, cur[m].y, cur[m].z, cur[m].w};
#pragma unroll
            for (int kk = 0; kk < 16; kk++) {
              const uint32_t c = (w[kk >> 2] >> ((kk & 3) * 8)) & 0xffu;
              const lut_t v    = my_lut[(m * 16 + kk) * 256 + c];
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
          if (wcount + 64u > wave_cap) {
            // make room: keep the k best of the buffer and tighten the wave's bound
            wave_sort_cap(my_cand, lane, wcount);
            if (wcount >= a.k) {
              wcount            = a.k;
              const uint32_t t2 = uint32_t(my_cand[a.k - 1] >> 32);
              thr               = t2 < thr ? t2 : thr;
            }
          }
          const bool pass2 = pass && okey <= thr;
          const unsigned long long mask2 = __ballot(pass2);
          const uint32_t below =
            __builtin_amdgcn_mbcnt_hi(uint32_t(mask2 >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask2), 0u));
          if (pass2) { my_cand[wcount + below] = (static_cast<unsigned long long>(okey) << 32) | (sample_off + i); }
          wcount += uint32_t(__popcll(mask2));
        }
        if (tile + WG < n_tiles) {
#pragma unroll
          for (int m = 0; m < NCH; m++) { cur[m] = ahead[m]; }
        }
      }
      // this wave's best candidates of the pair
      unsigned long long* out = a.out_keys + (uint64_t(my_d.slot) * WG + wig) * a.k;
      if (wcount >= a.k) {
        wave_sort_cap(my_cand, lane, wcount);  // only as wide as there are candidates
        wcount = a.k;
        if (lane == 0) { atomicMin(&a.query_kth[my_d.q], uint32_t(my_cand[a.k - 1] >> 32)); }
      }
      for (uint32_t t = lane; t < a.k; t += 64u) { out[t] = t < wcount ? my_cand[t] : kInvalidKey; }
    }

    if (!has_next) { break; }
    // first tile and bound of the next pair (arrive while the other waves finish and during the
    // next table construction)
    my_d = nxt_d;
    if (my_d.n_rows != 0) {
      const uint32_t r0 = wig * 64u + lane;
      load_tile(my_d.data, r0 < my_d.n_rows ? r0 : 0u, cur);
      pre_thr = a.query_kth[my_d.q];
    }
    quad = nxt_quad;
    lds_barrier_q();  // every wave is done with the tables; next staged terms are visible
  }
}

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
void launch_quad_instance(const scan_args& a, hipStream_t stream)
{
  constexpr int G = 4;
  using lut_t     = typename lut_traits<LUT>::storage;
  auto kernel     = scan_quad_kernel<NCH, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP, G>;
  const size_t smem = kQuadLdsBase + size_t(G) * NCH * 16 * 256 * sizeof(lut_t) +
                      size_t(G) * NCH * 16 * PQ_LEN * (IP ? 2 : 1) * 4 +
                      size_t(kQuadWaves) * quad_wave_cap(a.k) * 8;
  // per instance: the LDS limit is raised once, to the largest request of any k this kernel serves
  static const int attr_set = [&] {
    const size_t smem_max = smem + size_t(kQuadWaves) * (quad_wave_cap(kQuadMaxK) - quad_wave_cap(a.k)) * 8;
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(smem_max)));
    return 1;
  }();
  (void)attr_set;
  const int n_cu = device_cu_count();
  uint32_t grid = uint32_t(n_cu);
  if (a.n_pairs_dev == nullptr) {
    const uint32_t n_quads = (a.n_pairs + G - 1) / G;
    if (grid > n_quads) { grid = n_quads; }
    if (grid == 0) { return; }
  }
  kernel<<<grid, kQuadThreads, smem, stream>>>(a);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int NCH, int PQ_LEN, bool PER_CLUSTER>
bool launch_quad_types(const scan_args& a, hipStream_t s)
{
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (!ip) {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_16F) { launch_quad_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_quad_instance<NCH, PQ_LEN, LUT_FP8U, false, PER_CLUSTER, false>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_quad_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_quad_instance<NCH, PQ_LEN, LUT_FP8U, true, PER_CLUSTER, false>(a, s); return true; }
    }
  } else {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_16F) { launch_quad_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_quad_instance<NCH, PQ_LEN, LUT_FP8S, false, PER_CLUSTER, true>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_quad_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_quad_instance<NCH, PQ_LEN, LUT_FP8S, true, PER_CLUSTER, true>(a, s); return true; }
    }
  }
  return false;
}

template <int NCH, int PQ_LEN>
bool launch_quad_kind(const scan_args& a, hipStream_t s)
{
  return a.per_cluster ? launch_quad_types<NCH, PQ_LEN, true>(a, s) : launch_quad_types<NCH, PQ_LEN, false>(a, s);
}

}  // namespace

uint32_t scan_quad_keys_per_pair(const scan_args& a)
{
  if (!a.fused || a.pq_bits != 8 || a.k > kQuadMaxK) { return 0; }
  if (a.rot_dim != a.pq_dim * a.pq_len) { return 0; }
  if (a.lut_dtype != CUDA_R_16F && a.lut_dtype != CUDA_R_8U) { return 0; }
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  // four tables plus the staged terms must fit the 160 KB of LDS
  const size_t elem = a.lut_dtype == CUDA_R_16F ? 2 : 1;
  const size_t lds  = kQuadLdsBase + 4 * size_t(a.pq_dim) * 256 * elem + 4 * size_t(a.rot_dim) * (ip ? 2 : 1) * 4 +
                     size_t(kQuadWaves) * quad_wave_cap(a.k) * 8;
  if (lds > 160 * 1024) { return 0; }
  const bool shape = (a.pq_dim == 64 && a.pq_len == 2) || (a.pq_dim == 48 && a.pq_len == 2) ||
                     (a.pq_dim == 32 && a.pq_len == 4);
  return shape ? (kQuadWaves / 4) * a.k : 0;
}

bool launch_scan_quad(const scan_args& a, hipStream_t stream)
{
  if (scan_quad_keys_per_pair(a) == 0 || a.n_queries == 0 || a.desc == nullptr) { return false; }
  if (a.pq_dim == 64 && a.pq_len == 2) { return launch_quad_kind<4, 2>(a, stream); }
  if (a.pq_dim == 48 && a.pq_len == 2) { return launch_quad_kind<3, 2>(a, stream); }
  if (a.pq_dim == 32 && a.pq_len == 4) { return launch_quad_kind<2, 4>(a, stream); }
  return false;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
