/*
 * CU-wide LUT + code-scan kernel for 8-bit codes of any pq_dim that is a multiple of 32: the
 * organisation of scan_stream.hip (one persistent 1024-thread block per CU, eight waves that build
 * lookup tables next to eight that scan with them, a tile's lookups as one block of assembly) with
 * the table of a (query, probe) pair taken in slabs of 64 subspaces, so that it never has to fit
 * LDS whole.  Same arithmetic as the other scan kernels (compute_similarity of the reference:
 * create_lut_impl.cuh:16-79, compute_distances_impl.cuh:40-105, compute_score_impl.cuh:55-79; the
 * reference keeps the whole table in shared memory when it fits and in global memory otherwise,
 * ivf_pq_compute_similarity_impl.cuh:337-596).
 *
 *   - An iteration of the block is (two neighbouring pairs, row block, slab): the builders make the
 *     two 32 KB tables of the slab's 64 subspaces (32 in a last slab of half the size), the
 *     scanners add the slab's entries to the rows' sums.  A row's sum passes from slab to slab
 *     through LDS (4 bytes a row, 8192 rows a pair: longer lists are taken in row blocks, each with
 *     its tables built again), so the entries are added in subspace order exactly as a single pass
 *     over the whole row would add them.
 *   - L2 metrics: a tile of 64 rows none of which can still beat the query's bound is dropped for
 *     good (sums only grow): each scanner wave keeps a mask of its live tiles and, in later slabs,
 *     loads and sums those only.
 *   - The builders cannot keep the codebooks of every slab in registers: a builder thread owns two
 *     neighbouring codes of a quarter of the slab's subspaces and fetches those components from
 *     memory (L2) for every iteration, a few subspaces ahead of the arithmetic.
 *   - Everything else is scan_stream.hip's: entries as binary16 numbers in the form the scan adds,
 *     two vector instructions per lookup, four scanner waves per pair with their own candidate
 *     buffers, tables written between two barriers while no scanner gathers, blocks of one XCD on
 *     neighbouring pairs.
 */
#pragma once

#include "scan_stream_tile.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

constexpr uint32_t kSlabThreads   = 1024;
constexpr uint32_t kSlabPairs     = 2;   // pairs per iteration
constexpr uint32_t kSlabScanners  = 8;   // scanner waves (and as many builder waves)
constexpr uint32_t kSlabWG        = kSlabScanners / kSlabPairs;  // scanner waves per pair
constexpr uint32_t kSlabMaxK      = 128;
constexpr uint32_t kSlabSubs      = 64;    // subspaces per slab
constexpr uint32_t kSlabRows      = 8192;  // rows of a pair whose sums are kept between slabs
constexpr uint32_t kSlabTiles     = kSlabRows / 64u;           // tiles of a row block
constexpr uint32_t kSlabWaveTiles = kSlabTiles / kSlabWG;      // of which a scanner wave owns every fourth
static_assert(kSlabWaveTiles == 32, "a wave's live tiles are the bits of one word");

/* LDS map (bytes).  The two tables sit at multiples of 32 KB so that a table's address splits into
 * a 64 KB window (high half of the address register) and an immediate offset below 64 K:
 *   table of pair 0 at 0x08000, of pair 1 at 0x10000; the rows' sums behind them. */
constexpr uint32_t kSlabStageBase = 16;
constexpr uint32_t kSlabStageSlot = kSlabSubs * 8u * 2u * 4u;  // bytes per (buffer, pair): 64 subspaces x 8 dimensions x 2 terms
constexpr uint32_t kSlabCandBase  = kSlabStageBase + 4u * kSlabStageSlot;
constexpr uint32_t kSlabPartBase  = 0x18000;
constexpr uint32_t kSlabLdsOneSlab = 0x18000;
constexpr uint32_t kSlabLdsBytes   = kSlabPartBase + kSlabPairs * kSlabRows * 4u;
__host__ __device__ constexpr uint32_t slab_table_base(uint32_t g) { return g == 0 ? 0x08000u : 0x10000u; }
/** Candidate keys a wave buffers: room for k kept ones plus one tile of 64 new ones. */
inline __host__ __device__ uint32_t slab_wave_cap(uint32_t k) { return k <= 64u ? 128u : 192u; }
static_assert(kSlabCandBase % 8u == 0u && kSlabCandBase + kSlabScanners * 192u * 8u <= 0x08000u,
              "small buffers must end below the tables");
static_assert(kSlabLdsBytes <= 160u * 1024u, "the whole LDS of a CU");

template <int NCH_LAST, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
struct slab_kernel {
  using traits = lut_traits<LUT>;
  static constexpr uint32_t G  = kSlabPairs;
  static constexpr uint32_t WG = kSlabWG;
  // fp32 sums: entry * kEntryScale is added (one instruction: the binary16 entry is widened inside a
  // multiply-add); 8-bit tables hold half the decoded value
  static constexpr float kEntryScale = LUT == LUT_F16 ? 1.0f : 2.0f;
  static constexpr int TERMS = IP ? 2 : 1;
  static constexpr int FPS   = PQ_LEN * TERMS;  // staged floats per subspace
  // a table of 16-bit entries takes 64 subspaces (four 16-byte chunks of a row) in its 32 KB, one
  // of fp32 entries 32
  static constexpr bool WIDE     = LUT == LUT_F32;
  static constexpr int SCH       = WIDE ? 2 : 4;         // chunks of a whole slab
  static constexpr uint32_t SUBS = 16u * SCH;            // its subspaces
  // unsigned 8-bit tables keep the entry's code itself, a byte an entry, decoded by the scanners
  // (fewer bank conflicts in 256 bytes a subspace than in 512; see scan_stream.hip)
  static constexpr bool BYTE     = LUT == LUT_FP8U;
  static constexpr uint32_t SUB_BYTES = WIDE ? 1024u : (BYTE ? 256u : 512u);  // bytes of a subspace's 256 entries
  static_assert((NCH_LAST == 2 || NCH_LAST == 4) && NCH_LAST <= SCH, "pq_dim is a multiple of 32");
  static_assert(!(WIDE && OUT_HALF), "fp32 entries are summed in fp32");
  static_assert(kSlabSubs * FPS * 4u <= kSlabStageSlot, "staged terms of a slab must fit their slot");
  // staging elements (pair, dimension of the slab) per builder thread
  static constexpr uint32_t E = (G * kSlabSubs * PQ_LEN + 511u) / 512u;

  const scan_args& a;
  uint32_t n_pairs, n_quads, grid, lb, n_it;  // n_it: quads (two pairs) this block takes
  uint32_t lane, rw;                          // lane; index of the wave among the waves of its role (0..7)
  uint32_t n_slabs, nch_total;

  __device__ __forceinline__ uint32_t quad_of(uint32_t qi) const { return lb + qi * grid; }

  /* ---- the block's sequence of iterations: quads, their row blocks, the slabs of each ---- */
  struct walker {
    uint32_t qi, rb, s, n_rb;
  };
  static __device__ __forceinline__ uint32_t row_blocks(uint32_t rows)
  {
    return rows <= kSlabRows ? 1u : (rows + kSlabRows - 1u) / kSlabRows;
  }
  /** Moves on by one iteration; true when that is the first one of the next quad (whose n_rb the
   *  caller sets). */
  __device__ __forceinline__ bool step(walker& w) const
  {
    if (++w.s < n_slabs) { return false; }
    w.s = 0;
    if (++w.rb < w.n_rb) { return false; }
    w.rb = 0;
    w.qi++;
    return true;
  }

  /** The k best of the n >= k keys in a wave's buffer; as narrow as the keys allow. */
  __device__ __forceinline__ uint32_t select_keys(LDS_AS unsigned long long* buf, uint32_t n) const
  {
    if (n <= 64u) { return wave_select_keys<1>(buf, lane, n, a.k); }
    if (n <= 128u) { return wave_select_keys<2>(buf, lane, n, a.k); }
    return wave_select_keys<3>(buf, lane, n, a.k);
  }

  /* ------------------------------------ builders ------------------------------------ */

  /** What the builders need to know about the two pairs of a quad: which query and list (for the
   *  operands they fetch) and the row count.  Raw fields of the records: they are requested well
   *  before anything looks at them. */
  struct quad_info {
    // plain members, selected by value: an array indexed by a thread's pair number would be given
    // memory by the compiler
    uint32_t q0, q1, label0, label1, rows0, rows1;
    // g is 0 or 1 (arithmetic, not a choice between two members: that would become an address)
    __device__ __forceinline__ uint32_t q(uint32_t g) const { return q0 + g * (q1 - q0); }
    __device__ __forceinline__ uint32_t label(uint32_t g) const { return label0 + g * (label1 - label0); }
    __device__ __forceinline__ uint32_t n_rows(uint32_t g) const { return rows0 + g * (rows1 - rows0); }
  };
  static_assert(G == 2, "two pairs per iteration");
  __device__ __forceinline__ quad_info load_info(uint32_t qi) const
  {
    quad_info r{0, 0, 0, 0, 0, 0};
    if (qi < n_it) {  // uniform
      const uint32_t slot = quad_of(qi) * G;
      if (slot < n_pairs) {
        const pair_desc* d = a.desc + slot;
        r.q0               = d->q;
        r.label0           = d->label;
        r.rows0            = d->n_rows;
      }
      if (slot + 1u < n_pairs) {
        const pair_desc* d = a.desc + slot + 1u;
        r.q1               = d->q;
        r.label1           = d->label;
        r.rows1            = d->n_rows;
      }
    }
    return r;
  }
  static __device__ __forceinline__ uint32_t info_row_blocks(const quad_info& r)
  {
    return row_blocks(r.rows0 > r.rows1 ? r.rows0 : r.rows1);
  }

  /** Operands of one iteration in a builder thread's registers. */
  struct staged {
    float q[E], c[E];
    uint32_t label0, label1;  // the probed lists (per-cluster codebooks)
    uint32_t flags;  // bit g: pair g has rows in this row block; bit 2: last slab; bit 3: an iteration at all; slab << 4
    __device__ __forceinline__ bool live(uint32_t g) const { return ((flags >> g) & 1u) != 0u; }
    __device__ __forceinline__ bool last() const { return (flags & 4u) != 0u; }
    __device__ __forceinline__ bool valid() const { return (flags & 8u) != 0u; }
    __device__ __forceinline__ uint32_t slab() const { return flags >> 4; }
  };
  /** Runs fn(NCH) for the slab's chunk count: SCH, or NCH_LAST in a last slab. */
  template <typename Fn>
  static __device__ __forceinline__ void for_chunks(bool last, Fn fn)
  {
    if constexpr (NCH_LAST == SCH) {
      fn(std::integral_constant<int, SCH>{});
    } else {
      if (last) {
        fn(std::integral_constant<int, NCH_LAST>{});
      } else {
        fn(std::integral_constant<int, SCH>{});
      }
    }
  }

  /** ds_write_b32 at addr + IMM: the entries of two neighbouring codes of one subspace. */
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

  /** The thread's staging elements of a slab of NCH chunks: element x < E is (pair, dimension)
   *  number bt + 512 x of the slab's G * 16 NCH * PQ_LEN. */
  template <int NCH>
  __device__ __forceinline__ void fetch_terms(const quad_info& info, uint32_t bt, staged& f) const
  {
    constexpr uint32_t DIMS = 16u * NCH * PQ_LEN;  // rotated dimensions of the slab
    const uint32_t d0       = f.slab() * (SUBS * PQ_LEN);
#pragma unroll
    for (uint32_t x = 0; x < E; x++) {
      const uint32_t idx = bt + 512u * x;
      f.q[x]             = 0.0f;
      f.c[x]             = 0.0f;
      if (idx < G * DIMS) {
        const uint32_t g   = idx / DIMS;
        const uint32_t dim = d0 + (idx - g * DIMS);
        if (f.live(g)) {
          f.q[x] = a.rot_q[uint64_t(info.q(g)) * a.rot_dim + dim];
          f.c[x] = a.centers_rot[uint64_t(info.label(g)) * a.rot_dim + dim];
        }
      }
    }
  }
  template <int NCH>
  __device__ __forceinline__ static void stage_terms(uint32_t buffer, uint32_t bt, const staged& f)
  {
    constexpr uint32_t DIMS = 16u * NCH * PQ_LEN;
#pragma unroll
    for (uint32_t x = 0; x < E; x++) {
      const uint32_t idx = bt + 512u * x;
      if (idx < G * DIMS) {
        const uint32_t g   = idx / DIMS;
        const uint32_t dim = idx - g * DIMS;
        auto* dst = reinterpret_cast<LDS_AS float*>(uintptr_t(kSlabStageBase + (buffer * G + g) * kSlabStageSlot));
        if constexpr (!IP) {
          dst[dim] = f.q[x] - f.c[x];
        } else {
          dst[2 * dim]     = f.q[x];
          dst[2 * dim + 1] = f.c[x] * f.q[x];
        }
      }
    }
  }

  // subspaces whose codebook components a builder thread requests together (16 registers)
  static constexpr int GB = PQ_LEN == 1 ? 8 : PQ_LEN == 2 ? 4 : PQ_LEN <= 4 ? 2 : 1;
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  struct book_group {
    f32x2 v[GB][PQ_LEN];
  };
  /** Components (t, code) and (t, code + 1) of subspaces j .. j + GB - 1. */
  __device__ __forceinline__ book_group load_books(uint32_t j, uint32_t code) const
  {
    book_group b;
    const auto* base = reinterpret_cast<const GLOBAL_AS float*>(reinterpret_cast<uintptr_t>(a.pq_centers)) +
                       uint64_t(j) * (PQ_LEN * 256u) + code;
#pragma unroll
    for (int u = 0; u < GB; u++) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) { b.v[u][t] = *reinterpret_cast<const GLOBAL_AS f32x2*>(base + (u * PQ_LEN + t) * 256); }
    }
    return b;
  }

  /** The thread's table entries of an iteration (slab of NCH chunks; terms staged in `buffer`) into
   *  registers: nothing is written while the scanners gather. */
  template <int NCH>
  __device__ __forceinline__ void compute_entries(uint32_t buffer, uint32_t quarter, uint32_t code, const staged& f,
                                                  uint32_t (&entries)[G][16]) const
  {
    constexpr int QM = 4 * NCH;  // subspaces of a builder thread
    constexpr int NG = QM / GB;
    static_assert(QM % GB == 0, "whole groups");
    const uint32_t j_first = f.slab() * SUBS + quarter * uint32_t(QM);
    book_group bk[2];
    if constexpr (!PER_CLUSTER) { bk[0] = load_books(j_first, code); }
    // per-cluster codebooks: the components of the thread's two codes in the books of the two lists,
    // the same for every subspace
    f32x2 cb[PER_CLUSTER ? G : 1][PQ_LEN];
    if constexpr (PER_CLUSTER) {
#pragma unroll
      for (uint32_t g = 0; g < G; g++) {
#pragma unroll
        for (int t = 0; t < PQ_LEN; t++) {
          cb[g][t] = f32x2{0.0f, 0.0f};
          if (f.live(g)) {
            cb[g][t] = *reinterpret_cast<const GLOBAL_AS f32x2*>(
              reinterpret_cast<const GLOBAL_AS float*>(reinterpret_cast<uintptr_t>(a.pq_centers)) +
              (uint64_t(g == 0 ? f.label0 : f.label1) * PQ_LEN + t) * 256 + code);
          }
        }
      }
    }
    // the staged terms of the thread's subspaces: one address register per pair and the subspace in
    // the reads' offsets (as scalars the compiler would hold an address per subspace)
    uint32_t term_base[G];
#pragma unroll
    for (uint32_t g = 0; g < G; g++) {
      term_base[g] = kSlabStageBase + (buffer * G + g) * kSlabStageSlot + quarter * uint32_t(QM * FPS) * 4u;
      asm volatile("" : "+v"(term_base[g]));
    }
#pragma unroll
    for (int gi = 0; gi < NG; gi++) {
      if constexpr (!PER_CLUSTER) {
        if (gi + 1 < NG) { bk[(gi + 1) & 1] = load_books(j_first + uint32_t((gi + 1) * GB), code); }
      }
#pragma unroll
      for (int u = 0; u < GB; u++) {
        const int jj = gi * GB + u;
#pragma unroll
        for (uint32_t g = 0; g < G; g++) {
          if (!f.live(g)) { continue; }  // uniform
          const auto* term = reinterpret_cast<const LDS_AS float*>(uintptr_t(term_base[g])) + jj * FPS;
          float score[2] = {0.0f, 0.0f};
#pragma unroll
          for (int t = 0; t < PQ_LEN; t++) {
            float tq, tc = 0.0f;
            if constexpr (!IP) {
              tq = term[t];
            } else {
              tq = term[2 * t];
              tc = term[2 * t + 1];
            }
#pragma unroll
            for (int e = 0; e < 2; e++) {
              const float pqc = PER_CLUSTER ? cb[PER_CLUSTER ? g : 0][t][e] : bk[gi & 1].v[u][t][e];
              if constexpr (!IP) {
                float df = tq;
                df -= pqc;
                score[e] = fmaf(df, df, score[e]);
              } else {
                score[e] -= tc;
                score[e] = fmaf(-tq, pqc, score[e]);
              }
            }
          }
          if constexpr (WIDE) {
            entries[g][2 * jj]     = __float_as_uint(score[0]);
            entries[g][2 * jj + 1] = __float_as_uint(score[1]);
          } else {
            entries[g][jj] = pack_entries(score[0], score[1]);
          }
        }
      }
      // the requests stay where they are written: one group ahead of the arithmetic, no further
      asm volatile("" ::: "memory");
    }
  }

  /** ds_write_b64 at addr + IMM: the fp32 entries of two neighbouring codes of one subspace. */
  template <int IMM>
  __device__ __forceinline__ static void entries_write_wide(uint32_t addr, uint32_t e0, uint32_t e1)
  {
    static_assert(IMM >= 0 && IMM < 65536, "the write's offset field has 16 bits");
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 two = {e0, e1};
    asm volatile("ds_write_b64 %0, %1 offset:%2" : : "v"(addr), "v"(two), "n"(IMM) : "memory");
  }

  /** ... and from the registers into the tables, while no scanner reads:
   *  entry (j, code) of a slab's table at base + j * SUB_BYTES + code * (2 or 4). */
  template <int NCH, int jj = 0>
  __device__ __forceinline__ static void write_entries(uint32_t waddr, const uint32_t (&entries)[16])
  {
    if constexpr (jj < 4 * NCH) {
      if constexpr (WIDE) {
        entries_write_wide<jj * 1024>(waddr, entries[2 * jj], entries[2 * jj + 1]);
      } else {
        entries_write<jj * int(SUB_BYTES)>(waddr, entries[jj]);
      }
      write_entries<NCH, jj + 1>(waddr, entries);
    }
  }
  template <int NCH>
  __device__ __forceinline__ static void write_tables(uint32_t quarter, uint32_t code, const staged& f,
                                                      const uint32_t (&entries)[G][16])
  {
#pragma unroll
    for (uint32_t g = 0; g < G; g++) {
      if (!f.live(g)) { continue; }  // uniform
      write_entries<NCH>(slab_table_base(g) + quarter * uint32_t(4 * NCH) * SUB_BYTES + code * (WIDE ? 4u : (BYTE ? 1u : 2u)), entries[g]);
    }
  }

  __device__ __forceinline__ void run_builder() const
  {
    // a builder thread owns two neighbouring codebook entries (their table entries share a dword)
    // of a quarter of the slab's subspaces: the staged terms of a subspace serve both
    const uint32_t bt      = rw * 64u + lane;  // 0..511
    const uint32_t code    = (bt & 127u) * 2u;
    const uint32_t quarter = rw >> 1;          // wave-uniform

    // The front of the pipeline runs two iterations ahead of the scanners: `fi` holds the records of
    // its quad and `fin` those of the quad after (requested when the front entered its quad).
    walker fw{0, 0, 0, 1};
    quad_info fi  = load_info(0);
    quad_info fin = load_info(1);
    fw.n_rb       = info_row_blocks(fi);
    // operands of the front's iteration; the front moves on
    auto take = [&]() __attribute__((always_inline)) -> staged {
      staged f{};
      f.flags = 0u;
      if (fw.qi >= n_it) { return f; }
      f.flags = 8u | (fw.s << 4) | (fw.s + 1u == n_slabs ? 4u : 0u);
#pragma unroll
      for (uint32_t g = 0; g < G; g++) { f.flags |= fi.n_rows(g) > fw.rb * kSlabRows ? 1u << g : 0u; }
      for_chunks(f.last(), [&](auto nch) __attribute__((always_inline)) { fetch_terms<decltype(nch)::value>(fi, bt, f); });
      f.label0 = fi.label0;
      f.label1 = fi.label1;
      if (step(fw)) {
        fi      = fin;
        fw.n_rb = info_row_blocks(fi);
        fin     = load_info(fw.qi + 1u);
      }
      return f;
    };
    auto stage = [&](uint32_t buffer, const staged& f) __attribute__((always_inline)) {
      for_chunks(f.last(), [&](auto nch) __attribute__((always_inline)) { stage_terms<decltype(nch)::value>(buffer, bt, f); });
    };
    uint32_t entries[G][16];
    auto compute = [&](uint32_t buffer, const staged& f) __attribute__((always_inline)) {
      for_chunks(f.last(), [&](auto nch) __attribute__((always_inline)) { compute_entries<decltype(nch)::value>(buffer, quarter, code, f, entries); });
    };
    auto write = [&](const staged& f) __attribute__((always_inline)) {
      for_chunks(f.last(), [&](auto nch) __attribute__((always_inline)) { write_tables<decltype(nch)::value>(quarter, code, f, entries); });
    };

    staged cur_f = take();
    stage(0, cur_f);
    staged nxt_f = take();
    block_barrier();  // terms of iteration 0 visible
    compute(0, cur_f);
    if (nxt_f.valid()) { stage(1, nxt_f); }
    write(cur_f);
    block_barrier();  // tables of iteration 0 and terms of iteration 1 visible
    for (uint32_t it = 0;; it++) {
      // the scanners are working on iteration `it`; nxt_f holds the operands of it + 1 (their terms
      // are staged in buffer (it + 1) & 1)
      staged after_f = take();
      if (nxt_f.valid()) { compute((it + 1u) & 1u, nxt_f); }
      block_barrier();  // the scanners are through with the tables of iteration `it`
      if (nxt_f.valid()) { write(nxt_f); }
      // buffer it & 1 was read when the entries of iteration `it` were computed, which is over
      if (after_f.valid()) { stage(it & 1u, after_f); }
      const bool more = nxt_f.valid();
      nxt_f           = after_f;
      block_barrier();  // tables of iteration it + 1 and terms of iteration it + 2 visible
      if (!more) { break; }
    }
  }

  /* ------------------------------------ scanners ------------------------------------ */

  __device__ __forceinline__ pair_desc record(uint32_t qi, uint32_t g) const
  {
    // slots past the end read as an empty pair
    const uint32_t slot = quad_of(qi) * G + g;
    pair_desc d         = a.desc[slot < n_pairs ? slot : n_pairs - 1u];
    if (slot >= n_pairs) {
      d.n_rows = 0;
      d.slot   = 0xFFFFFFFFu;
    }
    return d;
  }
  /** The larger row count of the two pairs of the block's quad number qi (0 past the end). */
  __device__ __forceinline__ uint32_t quad_rows(uint32_t qi) const
  {
    uint32_t rows = 0;
    if (qi < n_it) {
#pragma unroll
      for (uint32_t g = 0; g < G; g++) {
        const uint32_t slot = quad_of(qi) * G + g;
        if (slot < n_pairs) {
          const uint32_t r = a.desc[slot].n_rows;
          rows             = r > rows ? r : rows;
        }
      }
    }
    return rows;
  }

  /** Chunk SCH * s of `row`; chunk m of the slab is 32 vectors further on each. */
  __device__ __forceinline__ const GLOBAL_AS u32x4* row_ptr(const uint8_t* list_data, uint32_t row, uint32_t s) const
  {
    return reinterpret_cast<const GLOBAL_AS u32x4*>(reinterpret_cast<uintptr_t>(list_data) +
                                                    uint64_t(row >> 5) * (nch_total * 512u) + uint64_t(row & 31u) * 16u +
                                                    uint64_t(s) * (uint32_t(SCH) * 512u));
  }
  template <int NCH>
  __device__ __forceinline__ static void load_tile(const GLOBAL_AS u32x4* ptr, u32x4 (&dst)[4])
  {
#pragma unroll
    for (int m = 0; m < NCH; m++) { dst[m] = ptr[m * 32]; }
  }

  /** Tiles wig, wig + 4, ... of row block rb of a list, as a mask of the wave's tile numbers. */
  static __device__ __forceinline__ uint32_t wave_tiles(uint32_t n_rows, uint32_t rb, uint32_t wig)
  {
    const uint32_t n_tiles = (n_rows + 63u) >> 6;
    const uint32_t first   = rb * kSlabTiles;
    if (n_tiles <= first + wig) { return 0u; }
    const uint32_t nt  = n_tiles - first < kSlabTiles ? n_tiles - first : kSlabTiles;
    const uint32_t cnt = (nt - wig + WG - 1u) / WG;
    return cnt >= 32u ? 0xFFFFFFFFu : (1u << cnt) - 1u;
  }

  template <int GI>
  __device__ __forceinline__ void run_scanner() const
  {
    constexpr int IMMG = GI == 0 ? 0x8000 : 0;
    // The scanners' instructions go first: their adds release the next lookups, and the LDS pipeline
    // they feed is the scarcest resource; the builders' arithmetic fills the slots they leave.
    __builtin_amdgcn_s_setprio(3);
    const uint32_t wig = rw & 3u;
    const uint32_t cap = slab_wave_cap(a.k);
    auto* my_cand      = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(kSlabCandBase)) + rw * cap;
    // sums of the pair's rows between slabs: row r of the row block at word r
    auto* part         = reinterpret_cast<LDS_AS uint32_t*>(uintptr_t(kSlabPartBase + uint32_t(GI) * kSlabRows * 4u)) + lane;
    // (byte entries: the constant of their decoding in place of the entries' factor)
    const float one    = opaque_float(BYTE ? __uint_as_float(0x38080000u) : kEntryScale);
    uint32_t one_u     = WIDE ? 2u : (BYTE ? 0u : 1u);  // a code shifted by this is its entry's offset in a subspace's table
    asm volatile("" : "+v"(one_u));

    // address registers of the lookups: the window of the group's table in the high halves
    uint32_t addr[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      addr[i] = (GI == 0 ? 0u : 1u) << 16;
      asm volatile("" : "+v"(addr[i]));
    }

    // codes of the first live tile of an iteration (pair d, row block rb, slab s)
    u32x4 cur[4], ahead[4];
    auto prefetch = [&](const pair_desc& d, uint32_t rb, uint32_t s, uint32_t live) __attribute__((always_inline)) {
      if (live == 0u) { return; }
      const uint32_t t0  = uint32_t(__builtin_ctz(live));
      const uint32_t r0  = (rb * kSlabTiles + wig + WG * t0) * 64u + lane;
      const auto* ptr    = row_ptr(d.data, r0 < d.n_rows ? r0 : 0u, s);
      for_chunks(s + 1u == n_slabs, [&](auto nch) __attribute__((always_inline)) { load_tile<decltype(nch)::value>(ptr, cur); });
    };

    // The record of the next quad's pair is requested when the wave enters the current one: nothing
    // should wait for a record, and no scalar load may be in flight while a tile's lookups count
    // theirs (every request below is followed by a block barrier, which waits for it).
    walker w{0, 0, 0, 1};
    pair_desc my_d     = record(0, GI);
    pair_desc nxt_d    = record(n_it > 1 ? 1 : 0, GI);
    w.n_rb             = row_blocks(quad_rows(0));
    uint32_t n_rb_next = row_blocks(quad_rows(1));
    uint32_t live      = wave_tiles(my_d.n_rows, 0, wig);
    prefetch(my_d, 0, 0, live);
    uint32_t pre_thr = my_d.n_rows != 0 ? a.query_kth[my_d.q] : 0xFFFFFFFFu;
    block_barrier();
    block_barrier();  // tables of iteration 0 are complete

    const bool cosine = a.metric == int(DistanceType::CosineExpanded);
    uint32_t thr = 0xFFFFFFFFu, wcount = 0;
    bool fresh = true;  // the first iteration of a pair
    while (w.qi < n_it) {
      const bool last     = w.s + 1u == n_slabs;
      const bool pair_end = last && w.rb + 1u == w.n_rb;
      if (fresh) {
        thr    = 0xFFFFFFFFu;
        wcount = 0;
      }
      if (my_d.slot != 0xFFFFFFFFu && live != 0u) {
        const uint32_t n_rows     = my_d.n_rows;
        const uint32_t sample_off = my_d.sample_off;
        const uint8_t* list_data  = my_d.data;
        const int64_t* list_ids   = a.filter_bits != nullptr ? a.inds_ptrs[my_d.label] : nullptr;
        const uint32_t rb = w.rb, s = w.s;
        // the wave's bound: a key, and the same as a score (no bound: +inf; NaN scores never pass);
        // the query's may have come down since the pair's last slab
        {
          const uint32_t t0 = uint32_t(__builtin_amdgcn_readfirstlane(int(pre_thr)));
          thr               = t0 < thr ? t0 : thr;
        }
        float thr_f = thr >= 0xFF800000u ? __uint_as_float(0x7F800000u) : unorder_f32(thr);
        // sums of an L2 scan are not negative: past the bound means past its bits
        uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
        // One tile (number t among the wave's): the codes in `now` are summed while those of the
        // wave's next live tile tn arrive in `next`.
        auto scan_tile = [&](auto nch_c, auto last_c, uint32_t t, uint32_t tn, const u32x4 (&now)[4], u32x4 (&next)[4]) __attribute__((always_inline)) {
          constexpr int NCH   = decltype(nch_c)::value;
          constexpr bool LAST = decltype(last_c)::value;
          const uint32_t i    = (rb * kSlabTiles + wig + WG * t) * 64u + lane;
          // requested without a condition (past the end: row 0 again), so that the wait for `now`
          // is known to leave exactly these loads in flight
          const uint32_t in = (rb * kSlabTiles + wig + WG * tn) * 64u + lane;
          load_tile<NCH>(row_ptr(list_data, in < n_rows ? in : 0u, s), next);
          bool valid = i < n_rows;
          if (list_ids != nullptr) {
            if (valid) {
              const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[i];
              valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
            }
          }
          const unsigned long long in_play = __builtin_amdgcn_ballot_w64(valid);
          LDS_AS uint32_t* my_part         = part + (wig + WG * t) * 64u;
          uint32_t start                   = 0u;
          if (s != 0u) { start = *my_part; }
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // see ST_FIRST
          const uint32_t sum_bits =
            stream_tile_sum<NCH, OUT_HALF, !IP, IMMG, WIDE, BYTE>(now, addr, one_u, one, stop_bits, in_play, start);
          if constexpr (!LAST) {
            bool keep = true;
            if constexpr (!IP) {
              uint32_t bits = sum_bits;
              if constexpr (OUT_HALF) { bits = __float_as_uint(float(__builtin_bit_cast(_Float16, uint16_t(sum_bits)))); }
              keep = (__builtin_amdgcn_ballot_w64(bits <= stop_bits) & in_play) != 0ull;
            }
            if (keep) {
              *my_part = sum_bits;
            } else {
              live &= ~(1u << t);
            }
          } else {
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
          }
        };
        // the wave's live tiles in turn; the two code buffers swap roles from tile to tile
        auto run_tiles = [&](auto nch_c, auto last_c) __attribute__((always_inline)) {
          uint32_t m = live;
          uint32_t t = uint32_t(__builtin_ctz(m));
          m &= m - 1u;
          for (;;) {
            uint32_t tn = m != 0u ? uint32_t(__builtin_ctz(m)) : t;
            scan_tile(nch_c, last_c, t, tn, cur, ahead);
            if (m == 0u) { break; }
            t = tn;
            m &= m - 1u;
            tn = m != 0u ? uint32_t(__builtin_ctz(m)) : t;
            scan_tile(nch_c, last_c, t, tn, ahead, cur);
            if (m == 0u) { break; }
            t = tn;
            m &= m - 1u;
          }
        };
        if (last) {
          run_tiles(std::integral_constant<int, NCH_LAST>{}, std::true_type{});
        } else {
          run_tiles(std::integral_constant<int, SCH>{}, std::false_type{});
        }
      }

      // the next iteration: its first tile and the query's bound arrive while the other waves finish
      walker n            = w;
      const bool new_quad = step(n);
      if (new_quad) { n.n_rb = n_rb_next; }
      const pair_desc done_d     = my_d;
      const uint32_t n_keys_done = wcount;
      if (n.qi < n_it) {
        if (new_quad) { my_d = nxt_d; }
        if (new_quad || n.rb != w.rb) { live = wave_tiles(my_d.n_rows, n.rb, wig); }
        prefetch(my_d, n.rb, n.s, live);
        if (my_d.n_rows != 0) { pre_thr = a.query_kth[my_d.q]; }
      }
      if (new_quad) {
        nxt_d     = record(n.qi + 1u < n_it ? n.qi + 1u : n.qi, GI);
        n_rb_next = row_blocks(quad_rows(n.qi + 1u));
      }
      fresh = new_quad;
      block_barrier();  // every scanner is through with this iteration's tables
      // While the builders write the next tables: this wave's best candidates of a finished pair go
      // out, and their k-th bounds the query from now on.
      if (pair_end && done_d.slot != 0xFFFFFFFFu) {
        uint32_t n_keys         = n_keys_done;
        unsigned long long* out = a.out_keys + (uint64_t(done_d.slot) * WG + wig) * a.k;
        if (n_keys >= a.k) {
          const uint32_t kth = select_keys(my_cand, n_keys);
          n_keys             = a.k;
          if (lane == 0) { atomicMin(&a.query_kth[done_d.q], kth); }
        }
        for (uint32_t t = lane; t < a.k; t += 64u) { out[t] = t < n_keys ? my_cand[t] : kInvalidKey; }
      }
      block_barrier();  // the builders have written the next ones
      w = n;
    }
  }
};

template <int NCH_LAST, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
__global__ __launch_bounds__(kSlabThreads) void scan_slab_kernel(scan_args a)
{
  using body = slab_kernel<NCH_LAST, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP>;
  const uint32_t tid = threadIdx.x;
  const uint32_t wid = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it scalar
  // the same in every lane: keep it (and everything derived from it) in scalar registers
  const uint32_t n_pairs = __builtin_amdgcn_readfirstlane(a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs);
  const uint32_t n_quads = (n_pairs + kSlabPairs - 1u) / kSlabPairs;
  const uint32_t grid    = gridDim.x;
  // Workgroups go to the XCDs in turn; the blocks of one XCD take a contiguous run of pairs.
  const uint32_t lb = (grid & 7u) == 0u ? (blockIdx.x & 7u) * (grid >> 3) + (blockIdx.x >> 3) : blockIdx.x;
  if (lb >= n_quads) { return; }  // whole block, before any barrier
  const uint32_t nch_total = a.pq_dim >> 4;
  body k{a, n_pairs, n_quads, grid, lb, (n_quads - lb + grid - 1u) / grid, tid & 63u,
         (wid & 3u) | ((wid >> 3) << 2), (a.pq_dim + body::SUBS - 1u) / body::SUBS, nch_total};
  // waves 0-3 and 8-11 build, 4-7 and 12-15 scan: two of each kind on every SIMD
  if (((wid >> 2) & 1u) == 0u) {
    k.run_builder();
  } else if ((k.rw >> 2) == 0u) {
    k.template run_scanner<0>();
  } else {
    k.template run_scanner<1>();
  }
}

template <int NCH_LAST, int PQ_LEN, int LUT, bool OUT_HALF, bool PER_CLUSTER, bool IP>
void launch_slab_instance(const scan_args& a, hipStream_t stream)
{
  auto kernel = scan_slab_kernel<NCH_LAST, PQ_LEN, LUT, OUT_HALF, PER_CLUSTER, IP>;
  // per instance: the whole LDS of a CU belongs to the one resident block
  static const int attr_set = [&] {
    // the kernel addresses LDS by the map above: the compiler must not have put anything there
    hipFuncAttributes attr{};
    CUVS_HIP_TRY(hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(kernel)));
    CUVS_EXPECTS(attr.sharedSizeBytes == 0, "scan_slab_kernel: %zu bytes of LDS allocated by the compiler",
                 size_t(attr.sharedSizeBytes));
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(kSlabLdsBytes)));
    return 1;
  }();
  (void)attr_set;
  uint32_t grid = uint32_t(device_cu_count());
  if (a.n_pairs_dev == nullptr) {
    const uint32_t n_quads = (a.n_pairs + kSlabPairs - 1) / kSlabPairs;
    if (grid > n_quads) { grid = n_quads; }
    if (grid == 0) { return; }
  }
  constexpr uint32_t subs = LUT == LUT_F32 ? 32u : 64u;  // of a slab
  const uint32_t lds      = a.pq_dim > subs ? kSlabLdsBytes : kSlabLdsOneSlab;
  kernel<<<grid, kSlabThreads, lds, stream>>>(a);
  CUVS_HIP_TRY(hipGetLastError());
}

template <int NCH_LAST, int PQ_LEN, bool PER_CLUSTER>
bool launch_slab_types(const scan_args& a, hipStream_t s)
{
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (!ip) {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_16F) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_F16, false, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_FP8U, false, PER_CLUSTER, false>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_F16, true, PER_CLUSTER, false>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_FP8U, true, PER_CLUSTER, false>(a, s); return true; }
    }
  } else {
    if (!a.out_half) {
      if (a.lut_dtype == CUDA_R_16F) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_F16, false, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_FP8S, false, PER_CLUSTER, true>(a, s); return true; }
    } else {
      if (a.lut_dtype == CUDA_R_16F) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_F16, true, PER_CLUSTER, true>(a, s); return true; }
      if (a.lut_dtype == CUDA_R_8U) { launch_slab_instance<NCH_LAST, PQ_LEN, LUT_FP8S, true, PER_CLUSTER, true>(a, s); return true; }
    }
  }
  return false;
}

/** All instances of one pq_len (a translation unit each). */
template <int PQ_LEN>
bool launch_slab_len(const scan_args& a, hipStream_t s)
{
  if (a.lut_dtype == CUDA_R_32F) {
    // fp32 entries: slabs of 32 subspaces, all of them whole; fp32 sums
    if (a.out_half) { return false; }
    const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
    if (a.per_cluster) {
      if (ip) {
        launch_slab_instance<2, PQ_LEN, LUT_F32, false, true, true>(a, s);
      } else {
        launch_slab_instance<2, PQ_LEN, LUT_F32, false, true, false>(a, s);
      }
    } else {
      if (ip) {
        launch_slab_instance<2, PQ_LEN, LUT_F32, false, false, true>(a, s);
      } else {
        launch_slab_instance<2, PQ_LEN, LUT_F32, false, false, false>(a, s);
      }
    }
    return true;
  }
  const bool half_last = (a.pq_dim & 63u) != 0u;  // a last slab of 32 subspaces
  if (a.per_cluster) {
    return half_last ? launch_slab_types<2, PQ_LEN, true>(a, s) : launch_slab_types<4, PQ_LEN, true>(a, s);
  }
  return half_last ? launch_slab_types<2, PQ_LEN, false>(a, s) : launch_slab_types<4, PQ_LEN, false>(a, s);
}

}  // namespace
}  // namespace cuvs::neighbors::ivf_pq::detail
