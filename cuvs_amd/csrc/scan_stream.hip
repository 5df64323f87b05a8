/*
 * CU-wide LUT + code-scan kernel for 8-bit codes, k <= 128 and fp16 / 8-bit tables: the kernel
 * that streams the probed lists in the benchmark configurations.  Same arithmetic as the other
 * scan kernels (compute_similarity of the reference: create_lut_impl.cuh:16-79,
 * compute_distances_impl.cuh:40-105, compute_score_impl.cuh:55-79); the organisation is a
 * producer / consumer split inside one persistent 1024-thread block per CU:
 *
 *   - 8 of the 16 waves build lookup tables, the other 8 scan codes with them, at the same time:
 *     while the scanners work through the two (query, probe) pairs of iteration i, the builders
 *     compute the entries of the two tables of iteration i + 1 into registers, and write them into
 *     the one set of tables between the two block barriers that end an iteration (LDS writes that
 *     mix with the scanners' gathers cost several times what they cost alone).  On every SIMD two
 *     waves of each kind share the issue slots, so the vector work of the table build fills the
 *     cycles in which the scanners wait for their LDS gathers and code loads;
 *   - a builder thread owns two neighbouring codebook entries of a quarter of the subspaces and keeps
 *     those codebook components in registers for the whole kernel; the two table entries of a
 *     subspace go out as one 32-bit write (the scanners spend their registers on code
 *     tiles instead: the two roles are separate loops, so neither pays for the other's state);
 *   - every table entry is stored as a binary16 number in the form the scan adds: the entry itself
 *     for fp16 tables; for 8-bit tables the decoded value decode(encode(score)), which the reference
 *     computes again at every lookup - as it is when the sums are binary16, and halved when they are
 *     fp32 (half of every decoded 8-bit value is a binary16 number, the largest ones themselves are
 *     not), the scan then adding twice the entry, which is exact;
 *   - a lookup is two vector instructions: the code byte is shifted into the low half of an address
 *     register by one sub-dword instruction (the high half holds the table's 64 KB window, the
 *     subspace's offset sits in the read's immediate field), and the entry is added;
 *   - four scanner waves share a pair; each keeps its own candidate buffer and bound, and writes
 *     its <= k best candidates of the pair (the per-query merge sees 4 k keys per pair);
 *   - blocks that run on one XCD take neighbouring pairs, which probe the same lists: a list's
 *     codes come from HBM once and are then served by that XCD's L2.
 */
#include "scan_stream_tile.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

constexpr uint32_t kStreamThreads  = 1024;
constexpr uint32_t kStreamPairs    = 2;  // pairs per iteration
constexpr uint32_t kStreamScanners = 8;  // scanner waves (and as many builder waves)
constexpr uint32_t kStreamWG       = kStreamScanners / kStreamPairs;  // scanner waves per pair
constexpr uint32_t kStreamMaxK     = 128;

/* LDS map (bytes).  The two tables sit at multiples of 32 KB so that a table's address splits
 * into a 64 KB window (high half of the address register) and an immediate offset below 64 K:
 *   table of pair 0 at 0x08000, of pair 1 at 0x10000. */
constexpr uint32_t kStreamLdsBytes  = 0x18000;
constexpr uint32_t kStreamStageBase = 16;               // 2 buffers x 2 pairs x 256 floats
constexpr uint32_t kStreamStageSlot = 256 * 4;          // bytes per (buffer, pair)
constexpr uint32_t kStreamCandBase  = 16 + 4 * kStreamStageSlot;
__host__ __device__ constexpr uint32_t stream_table_base(uint32_t g) { return g == 0 ? 0x08000u : 0x10000u; }

/** Candidate keys a wave buffers: room for k kept ones plus one tile of 64 new ones. */
inline __host__ __device__ uint32_t stream_wave_cap(uint32_t k) { return k <= 64u ? 128u : 192u; }
static_assert(kStreamCandBase % 8u == 0u && kStreamCandBase + kStreamScanners * 192u * 8u <= 0x08000u,
              "small buffers must end below the tables");


template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
struct stream_kernel {
  using traits = lut_traits<LUT>;
  using acc_t  = typename std::conditional<OUT_HALF, _Float16, float>::type;
  static constexpr int M              = NCH * 16;  // pq_dim
  static constexpr uint32_t ROT       = uint32_t(M) * PQ_LEN;
  static constexpr uint32_t n_diff    = ROT * (IP ? 2u : 1u);
  static constexpr uint32_t G         = kStreamPairs;
  static constexpr uint32_t WG        = kStreamWG;
  // fp32 sums: entry * kEntryScale is added (one instruction: the binary16 entry is widened inside a
  // multiply-add); 8-bit tables hold half the decoded value
  static constexpr float kEntryScale = LUT == LUT_F16 ? 1.0f : 2.0f;
  // Unsigned 8-bit tables (L2 metrics) keep the entry's 8-bit code itself, a byte an entry: the
  // scan's reads then fall into 256 bytes a subspace instead of 512 (fewer bank conflicts), the
  // table's writes are half as many bytes, and the builders skip the decoding; the scanners decode
  // with one shift-and-add per lookup.
  static constexpr bool BYTE            = LUT == LUT_FP8U;
  static constexpr uint32_t SUB_BYTES   = BYTE ? 256u : 512u;  // bytes of a subspace's 256 entries
  static constexpr uint32_t ENTRY_BYTES = BYTE ? 1u : 2u;
  static_assert(n_diff * 4u <= kStreamStageSlot, "staged terms of a pair must fit their slot");
  static_assert(ROT * G <= 512u, "one builder thread stages one (pair, dimension)");
  static_assert(uint32_t(M) * 512u <= 0x8000u, "a table must fit its 32 KB slot");

  const scan_args& a;
  uint32_t n_pairs, n_quads, grid, lb, n_it;
  uint32_t lane, rw;  // lane; index of the wave among the waves of its role (0..7)

  __device__ __forceinline__ pair_desc record(uint32_t quad, uint32_t g) const
  {
    // slots past the end read as an empty pair
    const uint32_t slot = quad * G + g;
    pair_desc d         = a.desc[slot < n_pairs ? slot : n_pairs - 1u];
    if (slot >= n_pairs) {
      d.n_rows = 0;
      d.slot   = 0xFFFFFFFFu;
    }
    return d;
  }
  __device__ __forceinline__ uint32_t quad_of(uint32_t it) const { return lb + it * grid; }

  /** The k best of the n >= k keys in a wave's buffer; as narrow as the keys allow. */
  __device__ __forceinline__ uint32_t select_keys(LDS_AS unsigned long long* buf, uint32_t n) const
  {
    if (n <= 64u) { return wave_select_keys<1>(buf, lane, n, a.k); }
    if (n <= 128u) { return wave_select_keys<2>(buf, lane, n, a.k); }
    return wave_select_keys<3>(buf, lane, n, a.k);
  }

  /* ------------------------------------ builders ------------------------------------ */

  /** What the builders need to know about the two pairs of an iteration: which query and list
   *  (for the operands they fetch) and the row count (nothing is built for an empty pair).  Raw
   *  fields of the records: they are requested an iteration before anything looks at them. */
  struct quad_info {
    uint32_t q[G], label[G], n_rows[G];
  };
  __device__ __forceinline__ quad_info load_info(uint32_t it) const
  {
    quad_info r;
#pragma unroll
    for (uint32_t g = 0; g < G; g++) {
      r.q[g]      = 0;
      r.label[g]  = 0;
      r.n_rows[g] = 0;
    }
    if (it < n_it) {  // uniform
#pragma unroll
      for (uint32_t g = 0; g < G; g++) {
        const uint32_t slot = quad_of(it) * G + g;
        if (slot < n_pairs) {
          const pair_desc* d = a.desc + slot;
          r.q[g]             = d->q;
          r.label[g]         = d->label;
          r.n_rows[g]        = d->n_rows;
        }
      }
    }
    return r;
  }

  struct staged {
    float q, c;
    float cb[PER_CLUSTER ? G : 1][PQ_LEN][2];  // per-cluster codebook components of the builder's two entries
    bool live[G];
  };

  /** One LDS write at addr + IMM: the entries of two neighbouring codes of one subspace. */
  template <int IMM>
  __device__ __forceinline__ static void entries_write(uint32_t addr, uint32_t two_entries)
  {
    static_assert(IMM >= 0 && IMM < 65536, "the write's offset field has 16 bits");
    if constexpr (BYTE) {
      asm volatile("ds_write_b16 %0, %1 offset:%2" : : "v"(addr), "v"(two_entries), "n"(IMM) : "memory");
    } else {
      asm volatile("ds_write_b32 %0, %1 offset:%2" : : "v"(addr), "v"(two_entries), "n"(IMM) : "memory");
    }
  }

  /** The entries of two scores side by side, the first in the low half. */
  __device__ __forceinline__ static uint32_t pack_entries(float s0, float s1)
  {
    if constexpr (LUT == LUT_F16) {
      // One rounding of each fp32 score to binary16.  The registers are made opaque first: the
      // compiler would otherwise fold the last multiply-add of a score into the conversion, which
      // rounds the exact product sum once instead of twice and changes values.
      asm volatile("" : "+v"(s0), "+v"(s1));
      typedef float f32x2 __attribute__((ext_vector_type(2)));
      typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
      const f16x2 h = __builtin_convertvector(f32x2{s0, s1}, f16x2);
      return __builtin_bit_cast(uint32_t, h);
    } else if constexpr (BYTE) {
      return uint32_t(traits::encode(s0)) | (uint32_t(traits::encode(s1)) << 8);
    } else {
      return uint32_t(table_entry<LUT, OUT_HALF>(s0)) | (uint32_t(table_entry<LUT, OUT_HALF>(s1)) << 16);
    }
  }

  static constexpr int TERMS   = IP ? 2 : 1;
  static constexpr int FPS     = PQ_LEN * TERMS;  // staged floats per subspace
  static constexpr int QM      = M / 4;           // subspaces of a builder thread
  static constexpr int GROUP   = 8 / FPS;         // subspaces whose terms make two 16-byte reads
  static constexpr int NGROUPS = QM / GROUP;
  static_assert(GROUP >= 1 && QM % GROUP == 0, "the subspaces of a builder thread split into whole groups");

  /** Entries of subspaces gi * GROUP .. + GROUP - 1 of the thread's quarter, for its two codes, from
   *  the subspaces' 8 staged floats. */
  template <int gi, int u = 0>
  __device__ __forceinline__ static void build_group(const float (&term)[8],
                                                     const float (&book)[PER_CLUSTER ? 1 : QM][PQ_LEN][2],
                                                     const float (&cb)[PQ_LEN][2], uint32_t (&entries)[QM])
  {
    if constexpr (u < GROUP) {
      constexpr int jj = gi * GROUP + u;
      float score[2]   = {0.0f, 0.0f};
#pragma unroll
      for (int e = 0; e < 2; e++) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          const float pqc = PER_CLUSTER ? cb[t][e] : book[PER_CLUSTER ? 0 : jj][t][e];
          if constexpr (!IP) {
            float df = term[u * FPS + t];
            df -= pqc;
            score[e] = fmaf(df, df, score[e]);
          } else {
            const float qv = term[u * FPS + 2 * t];
            score[e] -= term[u * FPS + 2 * t + 1];
            score[e] = fmaf(-qv, pqc, score[e]);
          }
        }
      }
      entries[jj] = pack_entries(score[0], score[1]);
      build_group<gi, u + 1>(term, book, cb, entries);
    }
  }

  template <int gi>
  __device__ __forceinline__ static void build_groups(const LDS_AS f32x4* terms, f32x4 (&cur4)[2],
                                                      const float (&book)[PER_CLUSTER ? 1 : QM][PQ_LEN][2],
                                                      const float (&cb)[PQ_LEN][2], uint32_t (&entries)[QM])
  {
    // the next group's terms are requested before this group is computed
    f32x4 nxt4[2];
    if constexpr (gi + 1 < NGROUPS) {
#pragma unroll
      for (int x = 0; x < 2; x++) { nxt4[x] = terms[(gi + 1) * 2 + x]; }
    }
    float term[8];
#pragma unroll
    for (int x = 0; x < 2; x++) {
      term[4 * x + 0] = cur4[x].x;
      term[4 * x + 1] = cur4[x].y;
      term[4 * x + 2] = cur4[x].z;
      term[4 * x + 3] = cur4[x].w;
    }
    build_group<gi>(term, book, cb, entries);
    if constexpr (gi + 1 < NGROUPS) {
#pragma unroll
      for (int x = 0; x < 2; x++) { cur4[x] = nxt4[x]; }
      build_groups<gi + 1>(terms, cur4, book, cb, entries);
    }
  }

  /** The thread's entries of one table go to LDS: entry (j, code) at base + j * SUB_BYTES + code * ENTRY_BYTES. */
  template <int jj = 0>
  __device__ __forceinline__ static void write_entries(uint32_t waddr, const uint32_t (&entries)[QM])
  {
    if constexpr (jj < QM) {
      entries_write<jj * int(SUB_BYTES)>(waddr, entries[jj]);
      write_entries<jj + 1>(waddr, entries);
    }
  }

  __device__ __forceinline__ void run_builder() const
  {
    // a builder thread owns two neighbouring codebook entries (their table entries share a dword)
    // of a quarter of the subspaces: the staged terms of a subspace serve both
    const uint32_t bt      = rw * 64u + lane;  // 0..511
    const uint32_t code    = (bt & 127u) * 2u;
    const uint32_t quarter = rw >> 1;          // wave-uniform
    float book[PER_CLUSTER ? 1 : QM][PQ_LEN][2];
    if constexpr (!PER_CLUSTER) {
#pragma unroll
      for (int jj = 0; jj < QM; jj++) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          const float2 two = *reinterpret_cast<const float2*>(
            a.pq_centers + ((quarter * QM + jj) * PQ_LEN + t) * 256 + code);
          book[jj][t][0] = two.x;
          book[jj][t][1] = two.y;
        }
      }
    } else {
      book[0][0][0] = 0.0f;
    }
    // operands of the pairs in `info`: the staging element (pair bt / ROT, dimension bt % ROT) and,
    // for per-cluster codebooks, this thread's components of both pairs' codebooks
    auto fetch = [&](const quad_info& info, staged& f) {
      f.q = 0.0f;
      f.c = 0.0f;
#pragma unroll
      for (uint32_t g = 0; g < G; g++) { f.live[g] = info.n_rows[g] != 0; }
      if (bt < ROT * G) {
        const uint32_t g   = bt / ROT;
        const uint32_t dim = bt - g * ROT;
        const bool live    = (g == 0 ? info.n_rows[0] : info.n_rows[G - 1]) != 0;
        if (live) {
          f.q = a.rot_q[uint64_t(g == 0 ? info.q[0] : info.q[G - 1]) * ROT + dim];
          f.c = a.centers_rot[uint64_t(g == 0 ? info.label[0] : info.label[G - 1]) * ROT + dim];
        }
      }
      if constexpr (PER_CLUSTER) {
#pragma unroll
        for (uint32_t g = 0; g < G; g++) {
#pragma unroll
          for (int t = 0; t < PQ_LEN; t++) {
            float2 two = make_float2(0.0f, 0.0f);
            if (info.n_rows[g] != 0) {
              two = *reinterpret_cast<const float2*>(a.pq_centers + (uint64_t(info.label[g]) * PQ_LEN + t) * 256 + code);
            }
            f.cb[g][t][0] = two.x;
            f.cb[g][t][1] = two.y;
          }
        }
      }
    };
    auto stage = [&](uint32_t buffer, const staged& f) {
      if (bt < ROT * G) {
        auto* dst = reinterpret_cast<LDS_AS float*>(
          uintptr_t(kStreamStageBase + (buffer * G + bt / ROT) * kStreamStageSlot));
        if constexpr (!IP) {
          dst[bt % ROT] = f.q - f.c;
        } else {
          dst[2 * (bt % ROT)]     = f.q;
          dst[2 * (bt % ROT) + 1] = f.c * f.q;
        }
      }
    };
    // the thread's table entries of iteration `it`, from the terms staged in buffer it & 1, into
    // registers: nothing is written while the scanners gather
    uint32_t entries[G][QM];
    auto compute = [&](uint32_t it, const staged& f) {
      const uint32_t buffer = it & 1u;
#pragma unroll
      for (uint32_t g = 0; g < G; g++) {
        if (!f.live[g]) { continue; }  // uniform
        const auto* terms = reinterpret_cast<const LDS_AS f32x4*>(
          uintptr_t(kStreamStageBase + (buffer * G + g) * kStreamStageSlot + quarter * uint32_t(QM * FPS) * 4u));
        f32x4 cur4[2];
#pragma unroll
        for (int x = 0; x < 2; x++) { cur4[x] = terms[x]; }
        build_groups<0>(terms, cur4, book, f.cb[PER_CLUSTER ? g : 0], entries[g]);
      }
    };
    // ... and from the registers into the tables, while no scanner reads
    auto write_tables = [&](const staged& f) {
#pragma unroll
      for (uint32_t g = 0; g < G; g++) {
        if (!f.live[g]) { continue; }  // uniform
        // entry (j, code) of the table at base + j * SUB_BYTES + code * ENTRY_BYTES; j = quarter * QM + jj
        write_entries<0>(stream_table_base(g) + quarter * uint32_t(QM) * SUB_BYTES + code * ENTRY_BYTES, entries[g]);
      }
    };

    staged cur_f{}, nxt_f{};
    quad_info info_a = load_info(0);
    quad_info info_b = load_info(1);
    fetch(info_a, cur_f);
    stage(0, cur_f);
    if (n_it > 1) { fetch(info_b, nxt_f); }
    info_a = load_info(2);  // always the records two iterations past the tables being built
    block_barrier();        // terms of iteration 0 visible
    compute(0, cur_f);
    if (n_it > 1) { stage(1, nxt_f); }
    write_tables(cur_f);
    block_barrier();  // tables of iteration 0 and terms of iteration 1 visible
    for (uint32_t it = 0; it < n_it; it++) {
      // the scanners are working on iteration `it`; nxt_f holds the operands of it + 1 (their terms
      // are staged), info_a the records of it + 2
      staged after_f{};
      const bool two_ahead = it + 2 < n_it;
      if (two_ahead) { fetch(info_a, after_f); }
      info_b = load_info(it + 3);
      if (it + 1 < n_it) { compute(it + 1, nxt_f); }
      block_barrier();  // the scanners are through with the tables of iteration `it`
      if (it + 1 < n_it) { write_tables(nxt_f); }
      // buffer it & 1 was read when the entries of iteration `it` were computed, which is over
      if (two_ahead) { stage(it & 1u, after_f); }
      nxt_f  = after_f;
      info_a = info_b;
      block_barrier();  // tables of iteration it + 1 and terms of iteration it + 2 visible
    }
  }

  /* ------------------------------------ scanners ------------------------------------ */

  /** Address of chunk 0 of `row`; chunk m is 32 vectors further on. */
  __device__ __forceinline__ static const GLOBAL_AS u32x4* row_ptr(const uint8_t* list_data, uint32_t row)
  {
    return reinterpret_cast<const GLOBAL_AS u32x4*>(
      reinterpret_cast<uintptr_t>(list_data) + uint64_t(row >> 5) * (NCH * 512u) + uint64_t(row & 31u) * 16u);
  }
  __device__ __forceinline__ static void load_tile(const GLOBAL_AS u32x4* ptr, u32x4 (&dst)[NCH])
  {
#pragma unroll
    for (int m = 0; m < NCH; m++) { dst[m] = ptr[m * 32]; }
  }

  template <int GI>
  __device__ __forceinline__ void run_scanner() const
  {
    constexpr int IMMG     = GI == 0 ? 0x8000 : 0;
    // The scanners' instructions go first: their adds release the next lookups, and the LDS pipeline
    // they feed is the scarcest resource; the builders' arithmetic fills the slots they leave.
    __builtin_amdgcn_s_setprio(3);
    const uint32_t wig     = rw & 3u;
    const uint32_t sw      = rw;  // scanner wave 0..7
    const uint32_t cap     = stream_wave_cap(a.k);
    auto* my_cand          = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(kStreamCandBase)) + sw * cap;
    // (byte entries: the constant of their decoding, and no shift from code to offset)
    const float one        = opaque_float(BYTE ? __uint_as_float(0x38080000u) : kEntryScale);
    uint32_t one_u         = BYTE ? 0u : 1u;
    asm volatile("" : "+v"(one_u));

    // address registers of the lookups: the window of the group's table in the high halves
    uint32_t addr[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      addr[i] = (GI == 0 ? 0u : 1u) << 16;
      asm volatile("" : "+v"(addr[i]));
    }

    // The record of the next iteration's pair is requested an iteration before it is looked at: the
    // first wait for codes after a request also waits for the request, and nothing should wait for
    // a record.
    pair_desc my_d  = record(quad_of(0), GI);
    pair_desc nxt_d = record(quad_of(n_it > 1 ? 1 : 0), GI);
    u32x4 cur[NCH], ahead[NCH];
    if (wig * 64u < my_d.n_rows) {
      const uint32_t r0 = wig * 64u + lane;
      load_tile(row_ptr(my_d.data, r0 < my_d.n_rows ? r0 : 0u), cur);
    }
    uint32_t pre_thr = my_d.n_rows != 0 ? a.query_kth[my_d.q] : 0xFFFFFFFFu;
    block_barrier();
    block_barrier();  // tables of iteration 0 are complete

    for (uint32_t it = 0; it < n_it; it++) {
      const bool has_next    = it + 1 < n_it;
      const pair_desc done_d = my_d;
      uint32_t n_keys        = 0;
      if (my_d.slot != 0xFFFFFFFFu) {
        const uint32_t n_rows     = my_d.n_rows;
        const uint32_t sample_off = my_d.sample_off;
        const uint8_t* list_data  = my_d.data;
        const int64_t* list_ids   = a.filter_bits != nullptr && n_rows != 0 ? a.inds_ptrs[my_d.label] : nullptr;
        const uint32_t n_tiles    = (n_rows + 63u) >> 6;
        // the wave's bound: a key, and the same as a score (no bound: +inf; NaN scores never pass)
        uint32_t thr = uint32_t(__builtin_amdgcn_readfirstlane(int(pre_thr)));
        float thr_f  = thr >= 0xFF800000u ? __uint_as_float(0x7F800000u) : unorder_f32(thr);
        // sums of an L2 scan are not negative: past the bound means past its bits
        uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
        uint32_t wcount    = 0;
        const bool cosine  = a.metric == int(DistanceType::CosineExpanded);
        // One tile: the codes in `now` are scanned while those of the wave's next tile arrive in `next`.
        auto scan_tile = [&](uint32_t tile, const u32x4 (&now)[NCH], u32x4 (&next)[NCH]) {
          const uint32_t i = tile * 64u + lane;
          // requested without a condition (past the end: row 0 again), so that the wait for `now`
          // is known to leave exactly these loads in flight
          const uint32_t in = i + WG * 64u;
          load_tile(row_ptr(list_data, in < n_rows ? in : 0u), next);
          bool valid = i < n_rows;
          if (list_ids != nullptr) {
            if (valid) {
              const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[i];
              valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
            }
          }
          const unsigned long long in_play = __builtin_amdgcn_ballot_w64(valid);
          const uint32_t sum_bits = stream_tile_sum<NCH, OUT_HALF, !IP, IMMG, false, BYTE>(now, addr, one_u, one, stop_bits, in_play);
          float score;
          if constexpr (OUT_HALF) {
            score = float(__builtin_bit_cast(_Float16, uint16_t(sum_bits)));
            if (cosine) { score = float(_Float16(__builtin_bit_cast(_Float16, uint16_t(sum_bits)) + _Float16(1))); }
          } else {
            score = __uint_as_float(sum_bits);
            if (cosine) { score += 1.0f; }
          }
          const unsigned long long mask = __builtin_amdgcn_ballot_w64(score <= thr_f) & in_play;
          if (mask != 0ull) {
            if (wcount + 64u > cap) {
              // make room (the buffer holds more than k keys): keep the k best and tighten the wave's bound
              const uint32_t t2 = select_keys(my_cand, wcount);
              wcount            = a.k;
              if (t2 < thr) {
                thr       = t2;
                thr_f     = unorder_f32(thr);
                stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
              }
            }
            const uint32_t okey            = order_f32(score);
            const bool pass                = ((mask >> lane) & 1ull) != 0ull && okey <= thr;
            const unsigned long long mask2 = __builtin_amdgcn_ballot_w64(pass);
            const uint32_t below =
              __builtin_amdgcn_mbcnt_hi(uint32_t(mask2 >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask2), 0u));
            if (pass) { my_cand[wcount + below] = (static_cast<unsigned long long>(okey) << 32) | (sample_off + i); }
            wcount += uint32_t(__popcll(mask2));
          }
        };
        // the two code buffers swap roles from tile to tile
        for (uint32_t tile = wig; tile < n_tiles; tile += 2u * WG) {
          scan_tile(tile, cur, ahead);
          if (tile + WG < n_tiles) { scan_tile(tile + WG, ahead, cur); }
        }
        n_keys = wcount;
      }

      // first tile and bound of the next pair: they arrive while the other waves finish
      if (has_next) {
        my_d = nxt_d;
        if (wig * 64u < my_d.n_rows) {
          const uint32_t r0 = wig * 64u + lane;
          load_tile(row_ptr(my_d.data, r0 < my_d.n_rows ? r0 : 0u), cur);
        }
        if (my_d.n_rows != 0) { pre_thr = a.query_kth[my_d.q]; }
      }
      nxt_d = record(quad_of(it + 2 < n_it ? it + 2 : it), GI);
      block_barrier();  // every scanner is through with this iteration's tables
      // While the builders write the next tables: this wave's best candidates of the pair go out,
      // and their k-th bounds the query from now on.
      if (done_d.slot != 0xFFFFFFFFu) {
        unsigned long long* out = a.out_keys + (uint64_t(done_d.slot) * WG + wig) * a.k;
        if (n_keys >= a.k) {
          const uint32_t kth = select_keys(my_cand, n_keys);
          n_keys             = a.k;
          if (lane == 0) { atomicMin(&a.query_kth[done_d.q], kth); }
        }
        for (uint32_t t = lane; t < a.k; t += 64u) { out[t] = t < n_keys ? my_cand[t] : kInvalidKey; }
      }
      block_barrier();  // the builders have written the next ones
    }
  }
};

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
__global__ __launch_bounds__(kStreamThreads) void scan_stream_kernel(scan_args a)
{
  using body = stream_kernel<NCH, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP>;
  const uint32_t tid = threadIdx.x;
  const uint32_t wid = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it scalar
  // the same in every lane: keep it (and everything derived from it) in scalar registers
  const uint32_t n_pairs = __builtin_amdgcn_readfirstlane(a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs);
  const uint32_t n_quads = (n_pairs + kStreamPairs - 1u) / kStreamPairs;
  const uint32_t grid    = gridDim.x;
  // Workgroups go to the XCDs in turn; the blocks of one XCD take a contiguous run of pairs.
  const uint32_t lb = (grid & 7u) == 0u ? (blockIdx.x & 7u) * (grid >> 3) + (blockIdx.x >> 3) : blockIdx.x;
  if (lb >= n_quads) { return; }  // whole block, before any barrier
  body k{a, n_pairs, n_quads, grid, lb, (n_quads - lb + grid - 1u) / grid, tid & 63u,
         (wid & 3u) | ((wid >> 3) << 2)};
  // waves 0-3 and 8-11 build, 4-7 and 12-15 scan: two of each kind on every SIMD
  if (((wid >> 2) & 1u) == 0u) {
    k.run_builder();
  } else if ((k.rw >> 2) == 0u) {
    k.template run_scanner<0>();
  } else {
    k.template run_scanner<1>();
  }
}

template <int NCH, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
void launch_stream_instance(const scan_args& a, hipStream_t stream)
{
  auto kernel = scan_stream_kernel<NCH, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP>;
  // per instance: the whole LDS of a CU belongs to the one resident block
  static const int attr_set = [&] {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(kStreamLdsBytes)));
    return 1;
  }();
  (void)attr_set;
  uint32_t grid = uint32_t(device_cu_count());
  if (a.n_pairs_dev == nullptr) {
    const uint32_t n_quads = (a.n_pairs + kStreamPairs - 1) / kStreamPairs;
    if (grid > n_quads) { grid = n_quads; }
    if (grid == 0) { return; }
  }
  kernel<<<grid, kStreamThreads, kStreamLdsBytes, stream>>>(a);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int NCH, int PQ_LEN, bool PER_CLUSTER>
bool launch_stream_types(const scan_args& a, hipStream_t s)
{
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (!ip) {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_16F) { launch_stream_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_stream_instance<NCH, PQ_LEN, LUT_FP8U, false, PER_CLUSTER, false>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_stream_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_stream_instance<NCH, PQ_LEN, LUT_FP8U, true, PER_CLUSTER, false>(a, s); return true; }
    }
  } else {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_16F) { launch_stream_instance<NCH, PQ_LEN, LUT_F16, false, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_stream_instance<NCH, PQ_LEN, LUT_FP8S, false, PER_CLUSTER, true>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_stream_instance<NCH, PQ_LEN, LUT_F16, true, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_stream_instance<NCH, PQ_LEN, LUT_FP8S, true, PER_CLUSTER, true>(a, s); return true; }
    }
  }
  return false;
}

template <int NCH, int PQ_LEN>
bool launch_stream_kind(const scan_args& a, hipStream_t s)
{
  return a.per_cluster ? launch_stream_types<NCH, PQ_LEN, true>(a, s) : launch_stream_types<NCH, PQ_LEN, false>(a, s);
}

}  // namespace

uint32_t scan_stream_keys_per_pair(const scan_args& a)
{
  if (!a.fused || a.pq_bits != 8 || a.k > kStreamMaxK) { return 0; }
  if (a.rot_dim != a.pq_dim * a.pq_len) { return 0; }
  if (a.lut_dtype != CUDA_R_16F && a.lut_dtype != CUDA_R_8U) { return 0; }
  const bool shape = (a.pq_dim == 64 && a.pq_len == 2) || (a.pq_dim == 48 && a.pq_len == 2) ||
                     (a.pq_dim == 32 && a.pq_len == 4) || (a.pq_dim == 32 && a.pq_len == 2);
  return shape ? kStreamWG * a.k : 0;
}

bool launch_scan_stream(const scan_args& a, hipStream_t stream)
{
  if (scan_stream_keys_per_pair(a) == 0 || a.n_queries == 0 || a.desc == nullptr) { return false; }
  if (a.pq_dim == 64 && a.pq_len == 2) { return launch_stream_kind<4, 2>(a, stream); }
  if (a.pq_dim == 48 && a.pq_len == 2) { return launch_stream_kind<3, 2>(a, stream); }
  if (a.pq_dim == 32 && a.pq_len == 4) { return launch_stream_kind<2, 4>(a, stream); }
  if (a.pq_dim == 32 && a.pq_len == 2) { return launch_stream_kind<2, 2>(a, stream); }
  return false;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
