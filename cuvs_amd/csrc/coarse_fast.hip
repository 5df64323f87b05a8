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
constexpr uint32_t kMinLine     = 32;  // PASS 1: group minima between two flushes: one 128-byte line of a query's row
constexpr uint32_t kCandFlushLists = 512;  // PASS 2: lists between two flushes of the candidates
constexpr uint32_t kMinRow      = kMinLine + 4u;  // floats per query in the staged minima (rows 144 bytes apart)

/** Shape of the GEMM by the padded dimension: MFMA tiles of 32 lists per list tile (NI), MFMA tiles
 *  of 32 queries per wave (NJ), blocks per CU.  A wave keeps its queries' whole rows in registers
 *  (K_PAD / 8 registers per query tile), and two buffers of a list tile sit in LDS
 *  (64 NI (K_PAD + 8) bytes): both shrink as the dimension grows. */
template <uint32_t K_PAD>
struct gemm_shape {
  static constexpr uint32_t NI     = K_PAD <= 256 ? 2 : 1;
  static constexpr uint32_t NJ     = K_PAD <= 512 ? 2 : 1;
  static constexpr uint32_t BLOCKS = K_PAD <= 128 ? 2 : 1;
};

/**
 * fp16 scores s' = alpha * (cn * qterm + dot16(c, q)) of a block's queries against a run of list
 * tiles.  Four waves, one per SIMD, each with 32 NJ of the queries and all 32 NI lists of a tile:
 * NI x NJ MFMA tiles of v_mfma_f32_32x32x16_f16 (each 16-byte read of the list operand out of LDS
 * feeds NJ products), the query operand in registers for the whole block.  Up to 128 dimensions two
 * blocks fit a CU, so that one block's matrix products run under the other's epilogue, staging
 * and barrier.  List tiles stream through two LDS buffers, the next tile's global loads in flight
 * while the current one is multiplied (one barrier per tile).  The norm term is the accumulators'
 * starting value.  PASS 1 keeps, per query, the minimum of every group of 32 lists; PASS 2 collects
 * the lists whose score is at or below the query's threshold.  Both results are staged in LDS by
 * the wave that owns the query and written out by that wave every so many tiles (the minima
 * as whole 128-byte lines; the candidates with one global atomic per query), without a barrier.
 * Both passes execute the same instructions up to the epilogue, so a list's score is the same
 * number in both.  K_PAD = padded dimension.
 */
template <int PASS, uint32_t K_PAD>
__global__ __launch_bounds__(kGemmThreads, gemm_shape<K_PAD>::BLOCKS) void coarse_f16_kernel(
  const _Float16* __restrict__ ch, const _Float16* __restrict__ qh, const float* __restrict__ cn,
  uint32_t n_lists, uint32_t n_queries, uint32_t q_rows, uint32_t n_list_tiles, uint32_t tiles_per_block, float alpha,
  float qterm, float* __restrict__ minima, uint32_t n_groups, const float* __restrict__ thr,
  uint32_t* __restrict__ cand_count, uint32_t* __restrict__ cand)
{
  constexpr uint32_t NI     = gemm_shape<K_PAD>::NI;
  constexpr uint32_t NJ     = gemm_shape<K_PAD>::NJ;
  constexpr uint32_t LT     = 32u * NI;          // lists per tile
  constexpr uint32_t QB     = 4u * 32u * NJ;     // queries per block
  constexpr uint32_t FLUSH1 = kMinLine / NI;     // PASS 1: list tiles between two flushes
  constexpr uint32_t FLUSH2 = kCandFlushLists / LT;
  constexpr uint32_t ROWB   = K_PAD * 2u + 16u;  // 16-byte reads of 32 consecutive rows hit all banks
  constexpr uint32_t CHUNKS = K_PAD / 8u;        // 16-byte chunks per row
  constexpr uint32_t PER_T  = LT * CHUNKS / kGemmThreads;  // chunks per thread and tile
  static_assert(LT * CHUNKS % kGemmThreads == 0 && PER_T >= 1 && PER_T <= 16, "a tile's chunks split evenly over the block");
  extern __shared__ __align__(16) unsigned char smem[];
  unsigned char* sa0 = smem;  // lists [2][LT][ROWB], two buffers
  float* scn         = reinterpret_cast<float*>(smem + 2u * LT * ROWB);  // [2][LT] norm terms
  uint32_t* lcount   = reinterpret_cast<uint32_t*>(scn + 2u * LT);       // PASS 2: [QB]
  uint32_t* lcand    = lcount + QB;                                      // PASS 2: [QB][kLocalCap]
  float* lmin        = reinterpret_cast<float*>(lcount);  // PASS 1: [QB][kMinRow] group minima
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = tid >> 6;  // the wave's quarter of the queries
  const uint32_t half = lane >> 5;
  const uint32_t q0   = blockIdx.y * QB;
  const uint32_t t0   = blockIdx.x * tiles_per_block;
  const uint32_t t1   = t0 + tiles_per_block < n_list_tiles ? t0 + tiles_per_block : n_list_tiles;
  const float neg_inf   = -__uint_as_float(0x7f800000u);
  const float inv_alpha = 1.0f / alpha;

  // this lane's queries inside the block (columns of the wave's query tiles); the packed queries
  // are padded to a multiple of 128 rows, a block's tail may lie beyond them.  The wave's query
  // operand never changes: it lives in registers.
  uint32_t qloc[NJ], q[NJ];
  v8h bq[NJ][K_PAD / 16u];
  float limit[NJ];
#pragma unroll
  for (uint32_t j = 0; j < NJ; j++) {
    limit[j]            = 0.0f;
    qloc[j]             = wid * (32u * NJ) + j * 32u + (lane & 31u);
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
      *reinterpret_cast<const uint4*>(ch + uint64_t(t0 * LT + crow[c]) * K_PAD + cpart[c] * 8u);
  }
  // per list: the norm term of the score, and for the padding lists a value no maximum picks
  if (tid < LT) {
    const uint32_t l = t0 * LT + tid;
    scn[tid]         = l < n_lists ? cn[l] * qterm : neg_inf;
  }
  if (PASS == 2) {
    for (uint32_t x = tid; x < QB; x += kGemmThreads) { lcount[x] = 0; }
  }
  __syncthreads();
  // Use the query operand once here, so that the compiler's wait for these loads sits here and not
  // inside the loop: there it would also wait for the staged loads below, which it does not count.
#pragma unroll
  for (uint32_t j = 0; j < NJ; j++) {
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
      const _Float16* src = ch + uint64_t(at * LT + crow[c]) * K_PAD + cpart[c] * 8u;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(st[c]) : "v"(src) : "memory");
    }
    // cn has coarse_pad(n_lists) entries: every thread loads one (most of the block a repeat)
    const float* src = cn + at * LT + (tid & (LT - 1u));
    asm volatile("global_load_dword %0, %1, off" : "=v"(sc) : "v"(src) : "memory");
  };
  auto arrived = [&](u32x4(&st)[PER_T], float& sc) __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(0)" : "+v"(sc) : : "memory");
#pragma unroll
    for (uint32_t c = 0; c < PER_T; c++) { asm volatile("" : "+v"(st[c]) : : "memory"); }
  };
  auto commit = [&](uint32_t tile, uint32_t buf, const u32x4(&st)[PER_T], float sc) __attribute__((always_inline)) {
    const uint32_t at  = tile < t1 ? tile : t1 - 1u;
    unsigned char* san = sa0 + buf * (LT * ROWB);
#pragma unroll
    for (uint32_t c = 0; c < PER_T; c++) {
      *reinterpret_cast<u32x4*>(san + crow[c] * ROWB + cpart[c] * 16u) = st[c];
    }
    if (tid < LT) { scn[buf * LT + tid] = at * LT + tid < n_lists ? sc * qterm : neg_inf; }
  };
  // products and epilogue of one tile out of LDS buffer `buf`
  auto multiply = [&](uint32_t tile, uint32_t buf) __attribute__((always_inline)) {
    const unsigned char* sa = sa0 + buf * (LT * ROWB);
    // element r of an MFMA tile: row (list) (r / 4) * 8 + (lane / 32) * 4 + r % 4, column (query) lane % 32
    v16f nv[NI];  // the norm terms of this lane's rows: where the sums start
#pragma unroll
    for (uint32_t i = 0; i < NI; i++) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const float4 t = *reinterpret_cast<const float4*>(scn + buf * LT + i * 32u + half * 4u + uint32_t(g) * 8u);
        nv[i][g * 4 + 0] = t.x;
        nv[i][g * 4 + 1] = t.y;
        nv[i][g * 4 + 2] = t.z;
        nv[i][g * 4 + 3] = t.w;
      }
    }
    v16f acc[NI][NJ];  // [list tile][query tile]
    // The list operand is read DEPTH steps ahead of the product that uses it, and the order is
    // pinned: left to itself the compiler, short of registers at the larger dimensions, reads each
    // step into the same registers and waits for it in front of its product (an LDS round trip
    // per product with nothing else to run on the SIMD).
    constexpr uint32_t KS    = K_PAD / 16u;
    constexpr uint32_t DEPTH = KS < 6u ? KS : (NI == 1 ? 6u : 4u);
    auto read_step = [&](uint32_t ks, v8h(&dst)[NI]) __attribute__((always_inline)) {
      const uint32_t kb = (ks * 16u + half * 8u) * 2u;  // byte offset of this lane's 8 values
#pragma unroll
      for (uint32_t i = 0; i < NI; i++) {
        dst[i] = *reinterpret_cast<const v8h*>(sa + (i * 32u + (lane & 31u)) * ROWB + kb);
      }
    };
    v8h a[DEPTH][NI];
#pragma unroll
    for (uint32_t d = 0; d < DEPTH; d++) { read_step(d, a[d]); }
#pragma unroll
    for (uint32_t ks = 0; ks < KS; ks++) {
#pragma unroll
      for (uint32_t i = 0; i < NI; i++) {
#pragma unroll
        for (uint32_t j = 0; j < NJ; j++) {
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[ks % DEPTH][i], bq[j][ks], ks == 0 ? nv[i] : acc[i][j], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (ks + DEPTH < KS) { read_step(ks + DEPTH, a[ks % DEPTH]); }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (PASS == 1) {
#pragma unroll
      for (uint32_t j = 0; j < NJ; j++) {
#pragma unroll
        for (uint32_t i = 0; i < NI; i++) {
          float best = neg_inf;
#pragma unroll
          for (int r = 0; r < 16; r++) { best = fmaxf(best, acc[i][j][r]); }  // NaN scores are ignored here and never pass the threshold
          // the lane 32 further on holds the tile's other 16 rows of this query
          best = fmaxf(best, __shfl_xor(best, 32, 64));
          if (half == 0) { lmin[qloc[j] * kMinRow + (tile % FLUSH1) * NI + i] = alpha * best; }
        }
      }
    } else {
      // bit (i * 16 + r) of miss[j]: that list is no candidate of query j.  The sign of v - limit is
      // shifted in element by element (two instructions an element), last element lowest.  A NaN
      // may land on either side: a NaN candidate sends the query to the plain path when it is
      // rescored.
      uint32_t hits[NJ];
      bool any = false;
#pragma unroll
      for (uint32_t j = 0; j < NJ; j++) {
        uint32_t m      = 0;
        const float lim = limit[j] * inv_alpha;  // alpha is -1 or -2: exact
#pragma unroll
        for (int i = int(NI) - 1; i >= 0; i--) {
#pragma unroll
          for (int r = 15; r >= 0; r--) { m = __builtin_amdgcn_alignbit(m, __float_as_uint(acc[i][j][r] - lim), 31); }
        }
        hits[j] = NI == 2 ? ~m : (~m) & 0xFFFFu;  // a single list tile fills the low 16 bits only
        any     = any || hits[j] != 0u;
      }
      if (any) {
#pragma unroll
        for (uint32_t j = 0; j < NJ; j++) {
          uint32_t h = hits[j];
          if (h == 0u) { continue; }
          uint32_t slot = atomicAdd(&lcount[qloc[j]], uint32_t(__popc(h)));
          while (h != 0u) {
            const uint32_t bit = uint32_t(__builtin_ctz(h));
            h &= h - 1u;
            const uint32_t row = (bit >> 4) * 32u + half * 4u + ((bit & 15u) >> 2) * 8u + (bit & 3u);
            const uint32_t s   = slot++;
            if (s < kLocalCap) { lcand[qloc[j] * kLocalCap + s] = tile * LT + row; }
          }
        }
      }
    }
  };
  // The wave writes out what it has staged for its queries since the last flush (its own LDS
  // writes, in order: no barrier).  PASS 1: the minima of tiles [first, tile], 16-byte parts (four
  // minima each: a block starts at a multiple of that many tiles) of one 128-byte line per query,
  // 8 queries an instruction.  PASS 2: a lane per query.
  auto flush = [&](uint32_t tile) __attribute__((always_inline)) {
    if (PASS == 1) {
      constexpr uint32_t TP = 4u / NI;                             // tiles per 16-byte part
      const uint32_t slot   = (tile % FLUSH1) / TP;                // the last part that has minima
      const uint32_t line   = tile - tile % FLUSH1;                // first tile of the line
      const uint32_t lo     = line < t0 ? (t0 - line) / TP : 0u;   // the block's first part of it
      const uint32_t part   = lane & 7u;
      // (all eight reads first and the stores after them measured 20 % slower for the whole kernel)
#pragma unroll
      for (uint32_t it = 0; it < 4u * NJ; it++) {
        const uint32_t ql = wid * (32u * NJ) + it * 8u + (lane >> 3);
        if (part >= lo && part <= slot && q0 + ql < n_queries) {
          *reinterpret_cast<float4*>(minima + uint64_t(q0 + ql) * n_groups + line * NI + part * 4u) =
            *reinterpret_cast<const float4*>(lmin + ql * kMinRow + part * 4u);
        }
      }
    } else {
      if (lane < 32u * NJ) {
        const uint32_t ql = wid * (32u * NJ) + lane;
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
    }
  };

  for (uint32_t tile = t0; tile < t1; tile++) {
    const uint32_t buf = (tile - t0) & 1u;
    issue(tile + 1u, sx, cx);
    multiply(tile, buf);
    if ((tile + 1u) % (PASS == 1 ? FLUSH1 : FLUSH2) == 0 || tile + 1u == t1) { flush(tile); }
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
  uint32_t n_probes, uint32_t* __restrict__ probes, uint8_t* __restrict__ fallback,
  float* __restrict__ probe_scores)
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
      if (probe_scores != nullptr) { probe_scores[uint64_t(q) * n_probes + rank] = unorder_f32(uint32_t(key >> 32)); }
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

/** The padded dimensions the GEMM has instances for. */
uint32_t coarse_fast_k_pad(uint32_t dim)
{
  for (uint32_t k : {64u, 128u, 256u, 384u, 512u, 768u}) {
    if (dim <= k) { return k; }
  }
  return 1024u;
}
uint32_t coarse_fast_max_dim() { return 1024u; }
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

  auto run_pass = [&](auto kpad) {
    constexpr uint32_t K_PAD = decltype(kpad)::value;
    using shape              = gemm_shape<K_PAD>;
    constexpr uint32_t LT = 32u * shape::NI, QB = 128u * shape::NJ, TP = 4u / shape::NI;
    auto k1 = coarse_f16_kernel<1, K_PAD>;
    auto k2 = coarse_f16_kernel<2, K_PAD>;
    // list tiles per block: the queries of a block are loaded once for all of them
    const uint32_t n_list_tiles = l_pad / LT;
    // A block costs about two tile-times of set-up besides its tiles, and the grid runs in rounds of
    // its blocks per CU: take the run length whose rounds x (tiles + 2) is smallest (the longest of
    // those: fewer blocks load the queries).
    const uint64_t n_slots   = uint64_t(device_cu_count()) * shape::BLOCKS;
    const uint32_t n_qblocks = (q_pad + QB - 1) / QB;
    uint32_t tiles_per_block = TP;
    uint64_t best_cost       = ~uint64_t(0);
    // (run lengths of whole 16-byte parts of the staged minima: four group minima)
    for (uint32_t t = TP; t <= n_list_tiles; t += TP) {
      const uint64_t blocks = uint64_t((n_list_tiles + t - 1) / t) * n_qblocks;
      const uint64_t rounds = (blocks + n_slots - 1) / n_slots;
      const uint64_t cost   = rounds * (t + 2);
      if (cost <= best_cost) {
        best_cost       = cost;
        tiles_per_block = t;
      }
    }
    dim3 grid((n_list_tiles + tiles_per_block - 1) / tiles_per_block, n_qblocks);
    // list tiles (two buffers), their norm terms, and the larger of the two passes' per-query areas
    const size_t smem = size_t(2) * LT * (K_PAD * 2 + 16) + 2 * LT * 4 +
                        std::max<size_t>(size_t(QB) * kMinRow * 4, size_t(QB) * (1 + kLocalCap) * 4);
    static const int limit_set = [&] {
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(k1), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
      CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(k2), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem)));
      return 1;
    }();
    (void)limit_set;
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
  switch (k_pad) {
    case 64: run_pass(std::integral_constant<uint32_t, 64>{}); break;
    case 128: run_pass(std::integral_constant<uint32_t, 128>{}); break;
    case 256: run_pass(std::integral_constant<uint32_t, 256>{}); break;
    case 384: run_pass(std::integral_constant<uint32_t, 384>{}); break;
    case 512: run_pass(std::integral_constant<uint32_t, 512>{}); break;
    case 768: run_pass(std::integral_constant<uint32_t, 768>{}); break;
    case 1024: run_pass(std::integral_constant<uint32_t, 1024>{}); break;
    default: CUVS_EXPECTS(false, "the two-precision probe selection takes dim <= 1024");
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
      coarse_rescore_kernel<float><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const float*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback, a.probe_scores);
      coarse_exact_rows_kernel<float><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const float*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
    case elem_type::f16:
      coarse_rescore_kernel<_Float16><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const _Float16*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback, a.probe_scores);
      coarse_exact_rows_kernel<_Float16><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const _Float16*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
    case elem_type::i8:
      coarse_rescore_kernel<int8_t><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const int8_t*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback, a.probe_scores);
      coarse_exact_rows_kernel<int8_t><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const int8_t*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
    default:
      coarse_rescore_kernel<uint8_t><<<a.n_queries, rthreads, rsmem, stream>>>(static_cast<const uint8_t*>(a.queries), a.centers, a.dim, a.dim_ext, qterm, alpha, a.cand_count, a.cand, a.n_probes, a.probes, a.fallback, a.probe_scores);
      coarse_exact_rows_kernel<uint8_t><<<a.n_queries, 256, xsmem, stream>>>(static_cast<const uint8_t*>(a.queries), a.centers, a.n_lists, a.dim, a.dim_ext, qterm, alpha, a.fallback, a.scores);
      break;
  }
  CUVS_HIP_TRY(hipGetLastError());
  // the flagged queries (normally none) take the plain selection over their exact rows
  launch_select_probes(a.scores, a.n_queries, a.n_lists, a.n_probes, a.probes, stream, a.fallback);
}

}  // namespace cuvs::neighbors::ivf_pq::detail
