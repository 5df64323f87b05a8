/*
 * Probe selection in two precisions, with the results of the fp32 path.
 *
 * select_clusters (cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:60-168) scores every centre for every
 * query in fp32 and keeps the n_probes best.  The fp32 contraction is most of that cost, and all of
 * it is spent on centres that are nowhere near the best.  Here the contraction runs on the fp16
 * matrix cores first (centres rounded to binary16, products exact, fp32 accumulation), with a
 * rigorous bound E_q on how far such a score can be from the fp32 one; every centre whose fp16
 * score is within 2 E_q of (an upper bound of) the n_probes-th smallest fp16 score is kept as a
 * candidate, which provably includes the fp32 path's n_probes best; the candidates - a few more
 * than n_probes - are then scored by the fp32 path's own arithmetic (one FMA chain over ascending
 * dimensions) and ordered by (score, list).  The probes are bit for bit those of the fp32 path.
 *
 *   pass 1  fp16 scores; per query the minimum of every group of 32 lists      (no score matrix)
 *   bound   T_q = n_probes-th smallest of those minima (at least n_probes scores are <= T_q),
 *           thr_q = T_q + 2 E_q
 *   pass 2  the same fp16 scores again; lists with score <= thr_q are appended to the query's
 *           candidate list
 *   rescore exact fp32 score of every candidate, rank, write the probes; a query with more
 *           candidates than fit (or fewer than n_probes: non-finite input) is flagged and goes
 *           through the plain fp32 path afterwards
 *
 * Why the candidates suffice: let s be fp32-path scores, s' the fp16 ones, |s - s'| <= E.  If t is
 * the n_probes-th smallest s, at most n_probes - 1 lists have s' < t - E, so the n_probes-th
 * smallest s' is >= t - E, and every list with s <= t has s' <= t + E <= (n_probes-th smallest s')
 * + 2E <= T + 2E.
 */
#include "scan_wave_select.cuh"

#include <mutex>

#include <algorithm>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kTile    = 64;   // lists per tile
constexpr uint32_t kQTile   = 256;  // queries per block: 4 waves x 64
constexpr uint32_t kSlab    = 64;   // the padded dimension is a multiple of this
constexpr uint32_t kCandCapF = 512;  // candidate slots per query (256 are used up to 128 probes)

template <typename T>
__device__ __forceinline__ float map_elem(T v);
template <>
__device__ __forceinline__ float map_elem<float>(float v) { return v; }
template <>
__device__ __forceinline__ float map_elem<_Float16>(_Float16 v) { return float(v); }
template <>
__device__ __forceinline__ float map_elem<int8_t>(int8_t v) { return float(v) * (1.0f / 128.0f); }
template <>
__device__ __forceinline__ float map_elem<uint8_t>(uint8_t v) { return float(v) * (1.0f / 256.0f); }

/** qh[q][d] = mapped query as binary16 (exact for these element types), zero padded to k_pad
 *  columns and q_pad rows; qnorm[q] = an upper bound of the query's Euclidean norm (of the
 *  unrounded values: float32 queries are the one type that binary16 does not hold exactly);
 *  qf[q][d] = the mapped query in fp32 (what the stages after the probe selection read). */
template <typename T>
__global__ void pack_queries_kernel(const T* __restrict__ in, uint32_t n_queries, uint32_t dim,
                                    uint32_t k_pad, _Float16* __restrict__ qh, float* __restrict__ qnorm,
                                    uint32_t* __restrict__ cand_count, uint8_t* __restrict__ fallback,
                                    float* __restrict__ qf)
{
  const uint32_t q    = blockIdx.x;
  const uint32_t lane = threadIdx.x;
  if (lane == 0) {
    // also start the query's candidate count and fall-back flag at zero
    cand_count[q] = 0;
    if (q < n_queries) { fallback[q] = 0; }
  }
  float ss            = 0.0f;
  for (uint32_t d = lane; d < k_pad; d += 64) {
    float v = 0.0f;
    if (q < n_queries && d < dim) {
      v = map_elem<T>(in[uint64_t(q) * dim + d]);
      if (qf != nullptr) { qf[uint64_t(q) * dim + d] = v; }
    }
    qh[uint64_t(q) * k_pad + d] = _Float16(v);
    ss                          = fmaf(v, v, ss);
  }
  for (int o = 32; o > 0; o >>= 1) { ss += __shfl_xor(ss, o); }
  if (lane == 0) { qnorm[q] = sqrtf(ss) * 1.0001f; }
}

/** ch[l][d] = centre as binary16, zero padded; cn[l] = the stored squared norm (column dim). */
__global__ void pack_centers_kernel(const float* __restrict__ centers, uint32_t n_lists, uint32_t dim,
                                    uint32_t dim_ext, uint32_t k_pad, _Float16* __restrict__ ch,
                                    float* __restrict__ cn, uint32_t* __restrict__ stats)
{
  const uint32_t l    = blockIdx.x;
  const uint32_t lane = threadIdx.x;
  float amax          = 0.0f;
  float ss            = 0.0f;
  for (uint32_t d = lane; d < k_pad; d += 64) {
    float v = 0.0f;
    if (l < n_lists && d < dim) { v = centers[uint64_t(l) * dim_ext + d]; }
    ch[uint64_t(l) * k_pad + d] = _Float16(v);
    amax                        = fmaxf(amax, fabsf(v));
    ss                          = fmaf(v, v, ss);
    if (v != v) { amax = __uint_as_float(0x7f800000u); }
  }
  for (int o = 32; o > 0; o >>= 1) {
    amax = fmaxf(amax, __shfl_xor(amax, o));
    ss += __shfl_xor(ss, o);
  }
  if (lane == 0) {
    const float nrm = l < n_lists ? centers[uint64_t(l) * dim_ext + dim] : 0.0f;
    cn[l]           = nrm;
    // non-negative floats order like their bit patterns: largest |element|, largest |stored norm|,
    // largest Euclidean length of a centre (rounded up)
    const float inf = __uint_as_float(0x7f800000u);
    atomicMax(&stats[0], __float_as_uint(amax));
    atomicMax(&stats[1], __float_as_uint(nrm == nrm ? fabsf(nrm) : inf));
    atomicMax(&stats[2], __float_as_uint(ss == ss ? sqrtf(ss) * 1.0001f : inf));
  }
}

constexpr uint32_t kGemmThreads = 256;
constexpr uint32_t kLocalCap    = 32;  // PASS 2: candidates a query may collect between two flushes before its block gives up
constexpr uint32_t kGroup       = 32;  // PASS 1: lists per group minimum (one MFMA tile's rows)
constexpr uint32_t kMinFlushTiles  = 16;  // PASS 1: list tiles between two flushes: 32 group minima, one 128-byte line of a query's row
constexpr uint32_t kCandFlushTiles = 8;   // PASS 2: list tiles (512 lists) between two flushes of the candidates
constexpr uint32_t kMinRow      = kMinFlushTiles * 2u + 4u;  // floats per query in the staged minima (rows 144 bytes apart)

/**
 * fp16 scores s' = alpha * (cn * qterm + dot16(c, q)) of a block's 256 queries against a run of
 * list tiles (64 lists each).  Four waves, one per SIMD, each with 64 of the queries and all 64
 * lists of a tile: four MFMA tiles of v_mfma_f32_32x32x16_f16 (each 16-byte read of the list
 * operand out of LDS feeds two products), the query operand in registers for the whole block.  Two
 * blocks fit a CU, so that one block's matrix products run under the other's epilogue, staging
 * and barrier.  List tiles stream through two LDS buffers, the next tile's global loads in flight
 * while the current one is multiplied (one barrier per tile).  The norm term is the accumulators'
 * starting value.  PASS 1 keeps, per query, the minimum of every group of 32 lists; PASS 2 collects
 * the lists whose score is at or below the query's threshold.  Both results are staged in LDS by
 * the wave that owns the query and written out by that wave every kFlushTiles tiles (the minima
 * as whole 128-byte lines; the candidates with one global atomic per query), without a barrier.
 * Both passes execute the same instructions up to the epilogue, so a list's score is the same
 * number in both.  K_PAD = padded dimension (64 or 128).
 */
template <int PASS, uint32_t K_PAD>
__global__ __launch_bounds__(kGemmThreads, 2) void coarse_f16_kernel(
  const _Float16* __restrict__ ch, const _Float16* __restrict__ qh, const float* __restrict__ cn,
  uint32_t n_lists, uint32_t n_queries, uint32_t q_rows, uint32_t n_list_tiles, uint32_t tiles_per_block, float alpha,
  float qterm, float* __restrict__ minima, uint32_t n_groups, const float* __restrict__ thr,
  uint32_t* __restrict__ cand_count, uint32_t* __restrict__ cand)
{
  constexpr uint32_t ROWB   = K_PAD * 2u + 16u;  // 16-byte reads of 32 consecutive rows hit all banks
  constexpr uint32_t CHUNKS = K_PAD / 8u;        // 16-byte chunks per row
  constexpr uint32_t PER_T  = kTile * CHUNKS / kGemmThreads;  // chunks per thread and tile (2 or 4)
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sa0 = smem;  // lists [2][64][ROWB], two buffers
  float* scn         = reinterpret_cast<float*>(smem + 2u * kTile * ROWB);  // [2][64] norm terms
  uint32_t* lcount   = reinterpret_cast<uint32_t*>(scn + 2u * kTile);       // PASS 2: [256]
  uint32_t* lcand    = lcount + kQTile;                                     // PASS 2: [256][kLocalCap]
  float* lmin        = reinterpret_cast<float*>(lcount);  // PASS 1: [256][kMinRow] group minima
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = tid >> 6;  // the wave's quarter of the queries (64)
  const uint32_t half = lane >> 5;
  const uint32_t q0   = blockIdx.y * kQTile;
  const uint32_t t0   = blockIdx.x * tiles_per_block;
  const uint32_t t1   = t0 + tiles_per_block < n_list_tiles ? t0 + tiles_per_block : n_list_tiles;
  const float neg_inf   = -__uint_as_float(0x7f800000u);
  const float inv_alpha = 1.0f / alpha;

  // this lane's two queries inside the block (columns of the wave's two query tiles); the packed
  // queries are padded to a multiple of 128 rows, a block's second half may lie beyond them.  The
  // wave's query operand never changes: it lives in registers.
  uint32_t qloc[2], q[2];
  v8h bq[2][K_PAD / 16u];
  float limit[2] = {0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < 2; j++) {
    qloc[j]             = wid * 64u + uint32_t(j) * 32u + (lane & 31u);
    q[j]                = q0 + qloc[j];
    const uint32_t q_rd = q[j] < q_rows ? q[j] : q_rows - 1u;
#pragma unroll
    for (uint32_t ks = 0; ks < K_PAD / 16u; ks++) {
      bq[j][ks] = *reinterpret_cast<const v8h*>(qh + uint64_t(q_rd) * K_PAD + ks * 16u + half * 8u);
    }
    // The epilogue works on v = norm term + dot; the score is alpha * v with alpha = -1 or -2, so
    // the smallest score of a group is alpha * (its largest v) and "score <= thr" is
    // "v >= thr / alpha", both exactly.  The threshold is only requested here: the first epilogue
    // is its first use, a tile of products later.
    if (PASS == 2) { limit[j] = q[j] < n_queries ? thr[q[j]] : neg_inf; }
  }

  // this thread's chunks of a tile: row and 16-byte part
  uint32_t crow[PER_T], cpart[PER_T];
#pragma unroll
  for (uint32_t c = 0; c < PER_T; c++) {
    const uint32_t chunk = tid + c * kGemmThreads;
    crow[c]              = chunk / CHUNKS;
    cpart[c]             = chunk % CHUNKS;
  }
  // the first list tile
#pragma unroll
  for (uint32_t c = 0; c < PER_T; c++) {
    *reinterpret_cast<uint4*>(sa0 + crow[c] * ROWB + cpart[c] * 16u) =
      *reinterpret_cast<const uint4*>(ch + uint64_t(t0 * kTile + crow[c]) * K_PAD + cpart[c] * 8u);
  }
  // per list: the norm term of the score, and for the padding lists a value no maximum picks
  if (tid < kTile) {
    const uint32_t l = t0 * kTile + tid;
    scn[tid]         = l < n_lists ? cn[l] * qterm : neg_inf;
  }
  if (PASS == 2) { lcount[tid] = 0; }
  __syncthreads();
  // Use the query operand once here, so that the compiler's wait for these loads sits here and not
  // inside the loop: there it would also wait for the staged loads below, which it does not count.
#pragma unroll
  for (int j = 0; j < 2; j++) {
#pragma unroll
    for (uint32_t ks = 0; ks < K_PAD / 16u; ks++) { asm volatile("" : "+v"(bq[j][ks])); }
  }

  // The next tile's loads go out at the top of an iteration and are written to the other LDS
  // buffer at its end.  They are written as instructions: as ordinary loads of read-only data the
  // compiler sinks them to their first use, behind the matrix products they are meant to overlap
  // (and as volatile loads it waits for each).  It does not count them, so the wait is explicit.
  // Tile numbers past the block's last tile repeat it (no branch around loads or stores).  (Loads
  // two tiles ahead, written to LDS half way through the next tile's products, measured the same:
  // the loop does not wait for them.)
  u32x4 sx[PER_T];
  float cx = 0.0f;
  auto issue = [&](uint32_t tile, u32x4(&st)[PER_T], float& sc) __attribute__((always_inline)) {
    const uint32_t at = tile < t1 ? tile : t1 - 1u;
#pragma unroll
    for (uint32_t c = 0; c < PER_T; c++) {
      const _Float16* src = ch + uint64_t(at * kTile + crow[c]) * K_PAD + cpart[c] * 8u;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(st[c]) : "v"(src) : "memory");
    }
    // cn has coarse_pad(n_lists) entries: every thread loads one (most of the block a repeat)
    const float* src = cn + at * kTile + (tid & (kTile - 1u));
    asm volatile("global_load_dword %0, %1, off" : "=v"(sc) : "v"(src) : "memory");
  };
  auto arrived = [&](u32x4(&st)[PER_T], float& sc) __attribute__((always_inline)) {
    if constexpr (PER_T == 4) {
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(st[0]), "+v"(st[1]), "+v"(st[2]), "+v"(st[3]), "+v"(sc) : : "memory");
    } else {
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(st[0]), "+v"(st[1]), "+v"(sc) : : "memory");
    }
  };
  auto commit = [&](uint32_t tile, uint32_t buf, const u32x4(&st)[PER_T], float sc) __attribute__((always_inline)) {
    const uint32_t at  = tile < t1 ? tile : t1 - 1u;
    unsigned char* san = sa0 + buf * (kTile * ROWB);
#pragma unroll
    for (uint32_t c = 0; c < PER_T; c++) {
      *reinterpret_cast<u32x4*>(san + crow[c] * ROWB + cpart[c] * 16u) = st[c];
    }
    if (tid < kTile) { scn[buf * kTile + tid] = at * kTile + tid < n_lists ? sc * qterm : neg_inf; }
  };
  // products and epilogue of one tile out of LDS buffer `buf`
  auto multiply = [&](uint32_t tile, uint32_t buf) __attribute__((always_inline)) {
    const unsigned char* sa = sa0 + buf * (kTile * ROWB);
    // element r of an MFMA tile: row (list) (r / 4) * 8 + (lane / 32) * 4 + r % 4, column (query) lane % 32
    v16f nv[2];  // the norm terms of this lane's rows: where the sums start
#pragma unroll
    for (int i = 0; i < 2; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const float4 t = *reinterpret_cast<const float4*>(scn + buf * kTile + uint32_t(i) * 32u + half * 4u + uint32_t(g) * 8u);
        nv[i][g * 4 + 0] = t.x;
        nv[i][g * 4 + 1] = t.y;
        nv[i][g * 4 + 2] = t.z;
        nv[i][g * 4 + 3] = t.w;
      }
    }
    v16f acc[2][2];  // [list tile][query tile]
#pragma unroll
    for (uint32_t ks = 0; ks < K_PAD / 16u; ks++) {
      const uint32_t kb = (ks * 16u + half * 8u) * 2u;  // byte offset of this lane's 8 values
      v8h a[2];
#pragma unroll
      for (int i = 0; i < 2; i++) {
        a[i] = *reinterpret_cast<const v8h*>(sa + (uint32_t(i) * 32u + (lane & 31u)) * ROWB + kb);
      }
#pragma unroll
      for (int i = 0; i < 2; i++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], bq[j][ks], ks == 0 ? nv[i] : acc[i][j], 0, 0, 0);
        }
      }
    }
    if (PASS == 1) {
#pragma unroll
      for (int j = 0; j < 2; j++) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
          float best = neg_inf;
#pragma unroll
          for (int r = 0; r < 16; r++) { best = fmaxf(best, acc[i][j][r]); }  // NaN scores are ignored here and never pass the threshold
          // the lane 32 further on holds the tile's other 16 rows of this query
          best = fmaxf(best, __shfl_xor(best, 32, 64));
          if (half == 0) { lmin[qloc[j] * kMinRow + (tile % kMinFlushTiles) * 2u + uint32_t(i)] = alpha * best; }
        }
      }
    } else {
      // bit (j * 32 + i * 16 + r) of `hits`: that list is a candidate of query j.  The sign of
      // v - limit is shifted in element by element (two instructions an element), last element
      // lowest: set bits are misses.  A NaN may land on either side: a NaN candidate sends the
      // query to the plain path when it is rescored.
      uint32_t miss[2];
#pragma unroll
      for (int j = 0; j < 2; j++) {
        uint32_t m      = 0;
        const float lim = limit[j] * inv_alpha;  // alpha is -1 or -2: exact
#pragma unroll
        for (int i = 1; i >= 0; i--) {
#pragma unroll
          for (int r = 15; r >= 0; r--) { m = __builtin_amdgcn_alignbit(m, __float_as_uint(acc[i][j][r] - lim), 31); }
        }
        miss[j] = m;
      }
      unsigned long long hits = ~((static_cast<unsigned long long>(miss[1]) << 32) | miss[0]);
      if (hits != 0) {
        uint32_t slot[2];
        slot[0] = atomicAdd(&lcount[qloc[0]], uint32_t(__popc(~miss[0])));
        slot[1] = atomicAdd(&lcount[qloc[1]], uint32_t(__popc(~miss[1])));
        while (hits != 0) {
          const uint32_t bit = uint32_t(__builtin_ctzll(hits));
          hits &= hits - 1u;
          const uint32_t j   = bit >> 5;
          const uint32_t row = ((bit >> 4) & 1u) * 32u + half * 4u + ((bit & 15u) >> 2) * 8u + (bit & 3u);
          const uint32_t s   = j ? slot[1]++ : slot[0]++;
          if (s < kLocalCap) { lcand[(j ? qloc[1] : qloc[0]) * kLocalCap + s] = tile * kTile + row; }
        }
      }
    }
  };
  // The wave writes out what it has staged for its 64 queries since the last flush (its own LDS
  // writes, in order: no barrier).  PASS 1: the minima of tiles [first, tile], 16-byte parts (two
  // tiles each: a block starts at an even tile) of one 128-byte line per query, 8 queries an
  // instruction.  PASS 2: a lane per query.
  auto flush = [&](uint32_t tile) __attribute__((always_inline)) {
    if (PASS == 1) {
      const uint32_t slot  = (tile % kMinFlushTiles) >> 1;
      const uint32_t line  = tile - tile % kMinFlushTiles;       // first tile of the line
      const uint32_t lo    = line < t0 ? (t0 - line) >> 1 : 0u;  // the block's first part of it
      const uint32_t part  = lane & 7u;
      // (all eight reads first and the stores after them measured 20 % slower for the whole kernel)
#pragma unroll
      for (uint32_t it = 0; it < 8; it++) {
        const uint32_t ql = wid * 64u + it * 8u + (lane >> 3);
        if (part >= lo && part <= slot && q0 + ql < n_queries) {
          *reinterpret_cast<float4*>(minima + uint64_t(q0 + ql) * n_groups + line * 2u + part * 4u) =
            *reinterpret_cast<const float4*>(lmin + ql * kMinRow + part * 4u);
        }
      }
    } else {
      const uint32_t ql = wid * 64u + lane;
      const uint32_t n  = lcount[ql];
      if (n != 0) {
        lcount[ql] = 0;
        if (q0 + ql < n_queries) {
          // more than the block can hold: push the query's count past the limit, it will be redone
          // by the plain path
          const uint32_t claim = n <= kLocalCap ? n : kCandCapF + 1u;
          const uint32_t base  = atomicAdd(&cand_count[q0 + ql], claim);
          if (n <= kLocalCap) {
            for (uint32_t e = 0; e < n; e++) {
              const uint32_t l = lcand[ql * kLocalCap + e];
              if (base + e < kCandCapF && l < n_lists) { cand[uint64_t(q0 + ql) * kCandCapF + base + e] = l; }
            }
          }
        }
      }
    }
  };

  for (uint32_t tile = t0; tile < t1; tile++) {
    const uint32_t buf = (tile - t0) & 1u;
    issue(tile + 1u, sx, cx);
    multiply(tile, buf);
    if ((tile + 1u) % (PASS == 1 ? kMinFlushTiles : kCandFlushTiles) == 0 || tile + 1u == t1) { flush(tile); }
    arrived(sx, cx);
    commit(tile + 1u, buf ^ 1u, sx, cx);
    // the barrier orders LDS traffic only (the staged tile); the flushes' global stores stay in
    // flight across it
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
}

/** thr[q] = (n_probes-th smallest of the query's group minima) + 2 E_q, rounded up.  One wave per
 *  query: the minima sit in registers as ordered keys (HELD per lane: 8 cover 16,384 lists, 64
 *  cover 131,072; more are re-read every round) and a round of the bitwise search counts with
 *  ballots, without LDS or barriers.  One probe (labelling rows during extend) needs no search:
 *  the threshold is the smallest minimum. */
template <uint32_t HELD>
__global__ __launch_bounds__(256) void coarse_threshold_kernel(
  const float* __restrict__ minima, uint32_t n_queries, uint32_t n_groups, uint32_t n_probes,
  const float* __restrict__ qnorm, float e_rel, float e_abs, float* __restrict__ thr)
{
  const uint32_t q    = blockIdx.x * 4u + (threadIdx.x >> 6);
  const uint32_t lane = threadIdx.x & 63u;
  if (q >= n_queries) { return; }
  const float* row = minima + uint64_t(q) * n_groups;
  uint32_t held[HELD];
#pragma unroll
  for (uint32_t h = 0; h < HELD; h++) {
    const uint32_t g = lane + h * 64u;
    const float v    = g < n_groups ? row[g] : __uint_as_float(0x7fc00000u);
    held[h]          = (v == v) ? order_f32(v) : 0xFFFFFFFFu;  // NaN and padding: above every probe but the last
  }
  // smallest ordered key K with count(keys <= K) >= n_probes, one bit at a time
  uint32_t prefix = 0;
  if (n_probes == 1u) {
    uint32_t lowest = 0xFFFFFFFFu;
#pragma unroll
    for (uint32_t h = 0; h < HELD; h++) { lowest = held[h] < lowest ? held[h] : lowest; }
    for (uint32_t g = HELD * 64u + lane; g < n_groups; g += 64u) {
      const float v    = row[g];
      const uint32_t k = (v == v) ? order_f32(v) : 0xFFFFFFFFu;
      lowest           = k < lowest ? k : lowest;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const uint32_t other = uint32_t(__shfl_xor(int(lowest), off, 64));
      lowest               = other < lowest ? other : lowest;
    }
    prefix = lowest;
  } else if (n_groups <= HELD * 64u) {
    // every minimum is in a register: radix selection over the bits in which they differ at all
    unsigned long long live[HELD];
#pragma unroll
    for (uint32_t h = 0; h < HELD; h++) { live[h] = __builtin_amdgcn_ballot_w64(lane + h * 64u < n_groups); }
    prefix = wave_kth_smallest<int(HELD)>(held, live, n_probes, lane);
  } else {
    for (int bit = 31; bit >= 0; bit--) {
      const uint32_t probe = prefix | ((1u << bit) - 1u);
      uint32_t n           = 0;
#pragma unroll
      for (uint32_t h = 0; h < HELD; h++) { n += uint32_t(__popcll(__builtin_amdgcn_ballot_w64(held[h] <= probe))); }
      for (uint32_t g0 = HELD * 64u; g0 < n_groups; g0 += 64u) {
        const uint32_t g = g0 + lane;
        const float v    = g < n_groups ? row[g] : __uint_as_float(0x7fc00000u);
        n += uint32_t(__popcll(__builtin_amdgcn_ballot_w64(v == v && order_f32(v) <= probe)));
      }
      if (n < n_probes) { prefix |= 1u << bit; }
    }
  }
  if (lane == 0) {
    const float t = unorder_f32(prefix);
    const float e = fmaf(e_rel, qnorm[q], e_abs);
    float bound   = t + 2.0f * e;
    bound += fabsf(bound) * 1e-6f;  // the additions above round to nearest
    thr[q] = bound;
  }
}

/** Exact fp32 score of every candidate by the fp32 path's arithmetic (one FMA chain over ascending
 *  dimensions, then the norm term), then the n_probes best in ascending (score, list) order.  One
 *  block per query, a lane per candidate.  A lane reading its own centre row costs a vector-cache
 *  lookup per lane and 16 bytes; here the 64 rows of a wave come in 32 dimensions at a time with
 *  whole 128-byte lines per 8 lanes, pass through the wave's own LDS area (rows 144 bytes apart),
 *  and every lane reads its row back; the next 32 dimensions are on their way meanwhile.  Nothing
 *  but the final ranking crosses waves. */
constexpr uint32_t kRescoreRow = 36;  // floats between the staged rows of a wave
template <typename T>
__global__ __launch_bounds__(512) void coarse_rescore_kernel(
  const T* __restrict__ queries, const float* __restrict__ centers, uint32_t dim, uint32_t dim_ext,
  float qterm, float alpha, const uint32_t* __restrict__ cand_count, const uint32_t* __restrict__ cand,
  uint32_t n_probes, uint32_t* __restrict__ probes, uint8_t* __restrict__ fallback)
{
  extern __shared__ __align__(16) unsigned char smem[];
  float* qf                 = reinterpret_cast<float*>(smem);  // [dim]
  unsigned long long* keys  = reinterpret_cast<unsigned long long*>(smem + ((dim * 4u + 15u) & ~15u));  // [threads]
  uint32_t* lcand           = reinterpret_cast<uint32_t*>(keys + blockDim.x);                           // [threads]
  float* stage_all          = reinterpret_cast<float*>(lcand + blockDim.x);  // [waves][64][kRescoreRow]
  const uint32_t q    = blockIdx.x;
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  // this thread's candidate is requested together with the count that says whether it has one
  // (tid < the candidate slots of a query: the address is always the query's own row)
  const uint32_t my_cand = cand[uint64_t(q) * kCandCapF + tid];
  const uint32_t n       = cand_count[q];
  // one candidate per thread: the block is as wide as the longest candidate list it accepts
  if (n > blockDim.x || n < n_probes) {
    if (tid == 0) { fallback[q] = 1; }
    return;
  }
  // The waves without a candidate leave at once (the barrier below counts the waves that are still
  // there): a typical query has ~70 candidates, and the slots of the idle waves let the next
  // queries' blocks start.
  const uint32_t n_active = (n + 63u) & ~63u;
  if (tid >= n_active) { return; }
  for (uint32_t d = tid; d < dim; d += n_active) { qf[d] = map_elem<T>(queries[uint64_t(q) * dim + d]); }
  lcand[tid] = tid < n ? my_cand : 0u;  // idle lanes of the last wave shadow list 0
  __syncthreads();
  float* stage = stage_all + (tid >> 6) * (64u * kRescoreRow);
  // lane -> (row, 16-byte piece) of the wave's k-th staging instruction: rows 8k .. 8k + 7
  const uint32_t piece = lane & 7u;
  const float* src[8];
#pragma unroll
  for (uint32_t k = 0; k < 8; k++) {
    src[k] = centers + uint64_t(lcand[(tid & ~63u) + k * 8u + (lane >> 3)]) * dim_ext + piece * 4u;
  }
  const float norm_term = centers[uint64_t(lcand[tid]) * dim_ext + dim];
  // two rounds of 32 dimensions are in flight while a third is multiplied
  float4 in[2][8];
  auto request = [&](uint32_t d0, float4(&dst)[8]) __attribute__((always_inline)) {
#pragma unroll
    for (uint32_t k = 0; k < 8; k++) {
      // a piece past the padded row is not read (rows are dim_ext floats, a multiple of 8)
      dst[k] = d0 + piece * 4u < dim_ext ? *reinterpret_cast<const float4*>(src[k] + d0) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
  };
  float acc = 0.0f;
  auto round = [&](uint32_t d0, float4(&cur)[8]) __attribute__((always_inline)) {
#pragma unroll
    for (uint32_t k = 0; k < 8; k++) {
      *reinterpret_cast<float4*>(stage + (k * 8u + (lane >> 3)) * kRescoreRow + piece * 4u) = cur[k];
    }
    if (d0 + 64 < dim) { request(d0 + 64, cur); }
    // the wave's own LDS writes, in order, before its reads of other lanes' words
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const float* row  = stage + lane * kRescoreRow;
    const uint32_t nd = dim - d0 < 32u ? dim - d0 : 32u;
    if (nd == 32u) {
#pragma unroll
      for (uint32_t x = 0; x < 8; x++) {
        const float4 v   = *reinterpret_cast<const float4*>(row + 4 * x);
        const uint32_t d = d0 + 4 * x;
        acc              = fmaf(v.x, qf[d], acc);
        acc              = fmaf(v.y, qf[d + 1], acc);
        acc              = fmaf(v.z, qf[d + 2], acc);
        acc              = fmaf(v.w, qf[d + 3], acc);
      }
    } else {
      for (uint32_t x = 0; x < nd; x++) { acc = fmaf(row[x], qf[d0 + x], acc); }
    }
    // ... and the reads before the next round's writes
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  };
  request(0, in[0]);
  if (32 < dim) { request(32, in[1]); }
  for (uint32_t d0 = 0; d0 < dim; d0 += 64) {
    round(d0, in[0]);
    if (d0 + 32 < dim) { round(d0 + 32, in[1]); }
  }
  unsigned long long key = kInvalidKey;
  if (tid < n) {
    acc           = fmaf(norm_term, qterm, acc);
    const float s = alpha * acc;
    key = (s != s) ? kInvalidKey : ((static_cast<unsigned long long>(order_f32(s)) << 32) | my_cand);
  }
  keys[tid] = key;
  __syncthreads();
  if (tid < n) {
    uint32_t rank = 0;
    for (uint32_t t = 0; t < n; t++) { rank += keys[t] < key ? 1u : 0u; }
    if (key == kInvalidKey) {
      fallback[q] = 1;  // a NaN score: let the plain path decide what it means
    } else if (rank < n_probes) {
      probes[uint64_t(q) * n_probes + rank] = uint32_t(key);
    }
  }
}

/** fp32 scores of every list for the flagged queries, into their rows of the score matrix. */
template <typename T>
__global__ __launch_bounds__(256) void coarse_exact_rows_kernel(
  const T* __restrict__ queries, const float* __restrict__ centers, uint32_t n_lists, uint32_t dim,
  uint32_t dim_ext, float qterm, float alpha, const uint8_t* __restrict__ flagged,
  float* __restrict__ scores)
{
  extern __shared__ __align__(16) unsigned char smem[];
  float* qf        = reinterpret_cast<float*>(smem);
  const uint32_t q = blockIdx.x;
  if (!flagged[q]) { return; }
  for (uint32_t d = threadIdx.x; d < dim; d += 256) { qf[d] = map_elem<T>(queries[uint64_t(q) * dim + d]); }
  __syncthreads();
  for (uint32_t l = threadIdx.x; l < n_lists; l += 256) {
    const float* c = centers + uint64_t(l) * dim_ext;
    float acc      = 0.0f;
    for (uint32_t d = 0; d < dim; d++) { acc = fmaf(c[d], qf[d], acc); }
    acc                               = fmaf(c[dim], qterm, acc);
    scores[uint64_t(q) * n_lists + l] = alpha * acc;
  }
}

}  // namespace

uint32_t coarse_fast_k_pad(uint32_t dim) { return (dim + kSlab - 1) / kSlab * kSlab; }
uint32_t coarse_fast_groups(uint32_t n_lists) { return coarse_pad(n_lists) / kGroup; }
uint32_t coarse_fast_cand_cap() { return kCandCapF; }

void launch_pack_centers_f16(const float* centers, uint32_t n_lists, uint32_t dim, uint32_t dim_ext,
                             _Float16* ch, float* cn, uint32_t* stats, hipStream_t stream)
{
  const uint32_t l_pad = coarse_pad(n_lists);
  CUVS_HIP_TRY(hipMemsetAsync(stats, 0, 16, stream));
  pack_centers_kernel<<<l_pad, 64, 0, stream>>>(centers, n_lists, dim, dim_ext, coarse_fast_k_pad(dim), ch, cn, stats);
  CUVS_HIP_TRY(hipGetLastError());
}

namespace {
template <typename K1, typename K2>
void lds_limit_once(int which, K1 k1, K2 k2, size_t smem)
{
  static std::once_flag flags[2];
  std::call_once(flags[which], [&] {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(k1), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(k2), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
  });
}
}  // namespace

void launch_coarse_fast(const coarse_fast_args& a, hipStream_t stream)
{
  const uint32_t q_pad = coarse_pad(a.n_queries);
  const uint32_t l_pad = coarse_pad(a.n_lists);
  const uint32_t k_pad = coarse_fast_k_pad(a.dim);
  const uint32_t n_groups = l_pad / kGroup;
  const float qterm    = a.ip_like ? 0.0f : -0.5f;
  const float alpha    = a.ip_like ? -1.0f : -2.0f;
  // |s - s'| <= |alpha| * [ (2^-11 + 9 (dim + 4) 2^-24) |q| Cmax + sqrt(dim) 2^-25 |q| + (dim + 4) 2^-24 * Nmax / 2 ],
  // inflated by 5 %: binary16 rounding of the centre elements (relative 2^-11, absolute 2^-25 below
  // the normal range), accumulation of dim + 1 terms in both chains, the epilogue's two roundings
  const float n_terms = float(a.dim + 4);
  const float two11 = 1.0f / 2048.0f, two24 = 1.0f / 16777216.0f;
  const float abs_alpha = a.ip_like ? 1.0f : 2.0f;
  // float32 queries are rounded to binary16 too: a second relative 2^-11 (and the product of the
  // two), and 2^-25 per element of a centre below binary16's normal range
  const bool rounded_q = a.type == elem_type::f32;
  const float q_round  = rounded_q ? two11 * 1.001f : 0.0f;
  const float e_rel = 1.05f * abs_alpha * ((two11 + q_round + 9.0f * n_terms * two24) * a.c_max + sqrtf(float(a.dim)) * two24 * 0.5f);
  const float e_abs = 1.05f * abs_alpha * (n_terms * two24 * 0.5f * a.n_max + (rounded_q ? sqrtf(float(a.dim)) * two24 * 0.5f * a.c_max : 0.0f));

  switch (a.type) {
    case elem_type::f32:
      pack_queries_kernel<float><<<q_pad, 64, 0, stream>>>(static_cast<const float*>(a.queries), a.n_queries, a.dim, k_pad, a.qh, a.qnorm, a.cand_count, a.fallback, a.qf);
      break;
    case elem_type::f16:
      pack_queries_kernel<_Float16><<<q_pad, 64, 0, stream>>>(static_cast<const _Float16*>(a.queries), a.n_queries, a.dim, k_pad, a.qh, a.qnorm, a.cand_count, a.fallback, a.qf);
      break;
    case elem_type::i8:
      pack_queries_kernel<int8_t><<<q_pad, 64, 0, stream>>>(static_cast<const int8_t*>(a.queries), a.n_queries, a.dim, k_pad, a.qh, a.qnorm, a.cand_count, a.fallback, a.qf);
      break;
    case elem_type::u8:
      pack_queries_kernel<uint8_t><<<q_pad, 64, 0, stream>>>(static_cast<const uint8_t*>(a.queries), a.n_queries, a.dim, k_pad, a.qh, a.qnorm, a.cand_count, a.fallback, a.qf);
      break;
  }
  CUVS_HIP_TRY(hipGetLastError());

  // list tiles per block: the queries of a block are loaded once for all of them
  const uint32_t n_list_tiles = l_pad / kTile;
  // A block costs about two tile-times of set-up besides its tiles, and the grid runs in rounds of
  // two blocks per CU: take the run length whose rounds x (tiles + 2) is smallest (the longest of
  // those: fewer blocks load the queries).
  const uint64_t n_slots   = uint64_t(device_cu_count()) * 2u;
  const uint32_t n_qblocks = (q_pad + kQTile - 1) / kQTile;
  uint32_t tiles_per_block = 2;
  uint64_t best_cost       = ~uint64_t(0);
  // (even run lengths: the group minima of two tiles share a 16-byte store)
  for (uint32_t t = 2; t <= n_list_tiles; t += 2) {
    const uint64_t blocks = uint64_t((n_list_tiles + t - 1) / t) * n_qblocks;
    const uint64_t rounds = (blocks + n_slots - 1) / n_slots;
    const uint64_t cost   = rounds * (t + 2);
    if (cost <= best_cost) {
      best_cost       = cost;
      tiles_per_block = t;
    }
  }
  dim3 grid((n_list_tiles + tiles_per_block - 1) / tiles_per_block, n_qblocks);
  auto run_pass = [&](auto k1, auto k2) {
    // list tiles (two buffers), their norm terms, and the larger of the two passes' per-query areas
    const size_t smem = size_t(2) * kTile * (k_pad * 2 + 16) + 2 * kTile * 4 +
                        std::max<size_t>(size_t(kQTile) * kMinRow * 4, size_t(kQTile) * (1 + kLocalCap) * 4);
    // a generic lambda has one body per pair of argument types, and the kernels of both K_PAD
    // values have the same type: the flag is keyed by K_PAD explicitly
    lds_limit_once(k_pad == 64 ? 0 : 1, k1, k2, smem);
    k1<<<grid, kGemmThreads, smem, stream>>>(a.ch, a.qh, a.cn, a.n_lists, a.n_queries, q_pad, n_list_tiles, tiles_per_block, alpha,
                                    qterm, a.minima, n_groups, nullptr, nullptr, nullptr);
    CUVS_HIP_TRY(hipGetLastError());
    if (n_groups <= 8u * 64u) {
      coarse_threshold_kernel<8><<<(a.n_queries + 3) / 4, 256, 0, stream>>>(a.minima, a.n_queries, n_groups, a.n_probes, a.qnorm, e_rel, e_abs, a.thr);
    } else if (n_groups <= 16u * 64u) {
      coarse_threshold_kernel<16><<<(a.n_queries + 3) / 4, 256, 0, stream>>>(a.minima, a.n_queries, n_groups, a.n_probes, a.qnorm, e_rel, e_abs, a.thr);
    } else {
      coarse_threshold_kernel<64><<<(a.n_queries + 3) / 4, 256, 0, stream>>>(a.minima, a.n_queries, n_groups, a.n_probes, a.qnorm, e_rel, e_abs, a.thr);
    }
    CUVS_HIP_TRY(hipGetLastError());
    k2<<<grid, kGemmThreads, smem, stream>>>(a.ch, a.qh, a.cn, a.n_lists, a.n_queries, q_pad, n_list_tiles, tiles_per_block, alpha,
                                    qterm, nullptr, n_groups, a.thr, a.cand_count, a.cand);
    CUVS_HIP_TRY(hipGetLastError());
  };
  if (k_pad == 64) {
    run_pass(coarse_f16_kernel<1, 64>, coarse_f16_kernel<2, 64>);
  } else {
    CUVS_EXPECTS(k_pad == 128, "the two-precision probe selection takes dim <= 128");
    run_pass(coarse_f16_kernel<1, 128>, coarse_f16_kernel<2, 128>);
  }
  // up to 128 probes about 1.4 x 128 candidates pass the threshold: 256 threads; 512 beyond
  // about 1.15 x n_probes candidates pass the threshold: 128 threads up to 64 probes, 256 up to
  // 128, 512 beyond (a query with more candidates than threads takes the plain path)
  const uint32_t rthreads = a.n_probes <= 64 ? 128u : (a.n_probes <= 128 ? 256u : 512u);
  const size_t rsmem      = ((size_t(a.dim) * 4 + 15) & ~size_t(15)) + size_t(rthreads) * 12 +
                       size_t(rthreads) * kRescoreRow * 4;
  const size_t xsmem = size_t(a.dim) * 4;
  CUVS_EXPECTS(rsmem <= 96 * 1024, "dim (%u) is too large for the two-precision probe selection", a.dim);
  if (rsmem > 48 * 1024) {
    static std::once_flag big_lds;
    std::call_once(big_lds, [&] {
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(coarse_rescore_kernel<float>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(coarse_rescore_kernel<_Float16>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(coarse_rescore_kernel<int8_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(coarse_rescore_kernel<uint8_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
    });
  }
  switch (a.type) {
    case elem_type::f32:
      coarse_rescore_kernel<float><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const float*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback);
      coarse_exact_rows_kernel<float><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const float*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
    case elem_type::f16:
      coarse_rescore_kernel<_Float16><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const _Float16*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback);
      coarse_exact_rows_kernel<_Float16><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const _Float16*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
    case elem_type::i8:
      coarse_rescore_kernel<int8_t><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const int8_t*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback);
      coarse_exact_rows_kernel<int8_t><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const int8_t*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
    default:
      coarse_rescore_kernel<uint8_t><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const uint8_t*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback);
      coarse_exact_rows_kernel<uint8_t><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const uint8_t*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
  }
  CUVS_HIP_TRY(hipGetLastError());
  // the flagged queries (normally none) take the plain selection over their exact rows
  launch_select_probes(a.scores, a.n_queries, a.n_lists, a.n_probes, a.probes, stream, a.fallback);
}

}  // namespace cuvs::neighbors::ivf_pq::detail
