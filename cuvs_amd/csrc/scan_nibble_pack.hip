/*
 * CU-wide LUT + code-scan kernel for 4-bit codes with binary16 tables (the sub-byte path of the
 * reference's compute_similarity kernel, cpp/src/neighbors/ivf_pq/detail/jit_lto_kernels/
 * compute_score_impl.cuh:13-79 with PqBits = 4; tables as in create_lut_impl.cuh:16-79).
 *
 * With 16 entries per subspace a lookup costs the LDS little (a wave's 64 lanes read inside one
 * 32-byte window), so the scan is bound by the vector instructions around the lookups, and the
 * kernel is built to need few of them:
 *
 *   - a lane scores two rows at a time, 64 apart: two independent chains of adds (binary16, or fp32
 *     through a multiply-add that widens the entry), so that one row's add is issued while the
 *     other's result is on its way.  Each row's entries are added
 *     one by one in subspace order, as the reference adds them.  (The two sums cannot share a
 *     register and a packed add: a 16-bit LDS read into one half of a register clears the other
 *     half on this hardware, whose register files are ECC protected.);
 *   - the table holds each entry as the binary16 number the reference's lookup decodes
 *     (decode(encode(score))), 32 bytes per subspace; a lookup's address register keeps the table's
 *     address in its upper three bytes, and one sub-dword shift writes 2 * nibble into its lowest
 *     byte (the nibbles of a code word are spread over the bytes of two masked copies first: three
 *     instructions per eight codes); the subspace's offset is the read's immediate;
 *   - a step of two 16-byte chunks per row (64 subspaces, 128 lookups) is one block of assembly
 *     with three groups of eight reads in flight while the oldest is added; an L2 scan looks at the
 *     query's bound after 8, 16, 32 and 48 subspaces and ends the step when none of the 128 rows can
 *     still win (early stop of compute_score in the reference), and has the next tile's first step
 *     on its way rather than this tile's next one.
 *
 * One persistent 1024-thread block per CU.  An iteration takes up to fifteen (query, probe) pairs:
 * all sixteen waves build the pairs' tables (a thread owns one codebook entry of every 64th
 * subspace and keeps those codebook components in registers), then each of the first fifteen waves
 * scans one pair against its table, with a candidate buffer and bound of its own, and writes the
 * pair's <= k best.  One wave per pair leaves no rows idle in a list's last tile but the last one's.
 */
#include "scan_wave_select.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kPackThreads   = 1024;
constexpr uint32_t kPackMaxPairs  = 15;    // pairs of an iteration: one scanner wave each
constexpr uint32_t kPackMaxK      = 64;
constexpr uint32_t kPackWaveCap   = 128;   // candidate keys a wave buffers: k kept ones and one tile's
constexpr uint32_t kPackCandBase  = 256;   // fifteen buffers of 1 KB
constexpr uint32_t kPackTableBase = 16384; // tables: pq_dim * 32 bytes each, 256-byte aligned
constexpr uint32_t kPackLdsBytes  = 160 * 1024;
constexpr uint32_t kPackStepBytes = 64 * 32;  // table bytes of the 64 subspaces of a step
static_assert(kPackCandBase + kPackMaxPairs * kPackWaveCap * 8u <= kPackTableBase, "candidate buffers end below the tables");

/* ---- one step (two chunks = 64 subspaces) of two rows, as one block of assembly ---- */
#define NP_MASKS(wa, wb)                                   \
  "v_and_b32_e32 %[evA], 0x0f0f0f0f, %[" #wa "]\n\t"       \
  "v_lshrrev_b32_e32 %[odA], 4, %[" #wa "]\n\t"            \
  "v_and_b32_e32 %[evB], 0x0f0f0f0f, %[" #wb "]\n\t"       \
  "v_lshrrev_b32_e32 %[odB], 4, %[" #wb "]\n\t"            \
  "v_and_b32_e32 %[odA], 0x0f0f0f0f, %[odA]\n\t"           \
  "v_and_b32_e32 %[odB], 0x0f0f0f0f, %[odB]\n\t"
#define NP_SDWA(a, m, b)                                                                                  \
  "v_lshlrev_b32_sdwa %[" #a "], %[one_u], %[" #m "] dst_sel:BYTE_0 dst_unused:UNUSED_PRESERVE src0_sel:DWORD " \
  "src1_sel:BYTE_" #b "\n\t"
#define NP_RD(v, a, j, i) "ds_read_u16 %[" #v "], %[" #a "] offset:" #j "*128+" #i "*32\n\t"
/* group j = subspaces 4 j .. 4 j + 3 of the step: the low (p0 = 0) or high (p0 = 2) four nibbles of a code word */
#define NP_ISSUE(j, V, p0, p1)                                                                              \
  NP_SDWA(aa0, evA, p0) NP_SDWA(aa1, odA, p0) NP_SDWA(aa2, evA, p1) NP_SDWA(aa3, odA, p1)                  \
  NP_SDWA(ab0, evB, p0) NP_SDWA(ab1, odB, p0) NP_SDWA(ab2, evB, p1) NP_SDWA(ab3, odB, p1)                  \
  NP_RD(V##a0, aa0, j, 0) NP_RD(V##a1, aa1, j, 1) NP_RD(V##a2, aa2, j, 2) NP_RD(V##a3, aa3, j, 3)          \
  NP_RD(V##b0, ab0, j, 0) NP_RD(V##b1, ab1, j, 1) NP_RD(V##b2, ab2, j, 2) NP_RD(V##b3, ab3, j, 3)
/* the two rows' sums are separate chains of adds: one proceeds while the other's result is on its way */
#define NP_ADD_H(acc, v) "v_add_f16_e32 %[" #acc "], %[" #acc "], %[" #v "]\n\t"
/* fp32 sums: the binary16 entry is widened inside a multiply-add by its factor (an exact product) */
#define NP_ADD_F(acc, v) "v_fma_mix_f32 %[" #acc "], %[" #v "], %[one], %[" #acc "] op_sel_hi:[1,0,0]\n\t"
#define NP_ADD4(ADD1, V)                                                              \
  ADD1(accA, V##a0) ADD1(accB, V##b0) ADD1(accA, V##a1) ADD1(accB, V##b1)             \
  ADD1(accA, V##a2) ADD1(accB, V##b2) ADD1(accA, V##a3) ADD1(accB, V##b3)
/* L2 sums only grow: when no row in play of either half is at or below the bound any more, the
 * step ends (the reads on their way are awaited and dropped).  Sums as the bits of a float. */
#define NP_CHECK_F                                     \
  "v_cmp_ge_u32_e32 vcc, %[stop], %[accA]\n\t"         \
  "s_and_b64 %[tmpA], vcc, %[validA]\n\t"              \
  "v_cmp_ge_u32_e32 vcc, %[stop], %[accB]\n\t"         \
  "s_and_b64 %[tmpB], vcc, %[validB]\n\t"              \
  "s_or_b64 %[tmpA], %[tmpA], %[tmpB]\n\t"             \
  "s_cbranch_scc0 .Lstep_done%=\n\t"
#define NP_CHECK_H                                     \
  "v_cvt_f32_f16_e32 %[chkA], %[accA]\n\t"             \
  "v_cvt_f32_f16_e32 %[chkB], %[accB]\n\t"             \
  "v_cmp_ge_u32_e32 vcc, %[stop], %[chkA]\n\t"         \
  "s_and_b64 %[tmpA], vcc, %[validA]\n\t"              \
  "v_cmp_ge_u32_e32 vcc, %[stop], %[chkB]\n\t"         \
  "s_and_b64 %[tmpB], vcc, %[validB]\n\t"              \
  "s_or_b64 %[tmpA], %[tmpA], %[tmpB]\n\t"             \
  "s_cbranch_scc0 .Lstep_done%=\n\t"
#define NP_NO_CHECK ""
#define NP_W15 "s_waitcnt lgkmcnt(15)\n\t"  /* of 24 reads in flight: the oldest group of eight has landed */
#define NP_W8 "s_waitcnt lgkmcnt(8)\n\t"
#define NP_W0 "s_waitcnt lgkmcnt(0)\n\t"
/* The sixteen groups of a step: three are in flight (sets x, y, z in turn) while the oldest is added;
 * the masked copies of code word d are made before its first group (2 d) is issued. */
#define NP_BODY(A, CHECK) \
  NP_MASKS(ca0, cb0) NP_ISSUE(0, x, 0, 1) NP_ISSUE(1, y, 2, 3) NP_MASKS(ca1, cb1) NP_ISSUE(2, z, 0, 1) \
  NP_W15 NP_ADD4(A, x) NP_ISSUE(3, x, 2, 3) \
  NP_W15 NP_ADD4(A, y) CHECK NP_MASKS(ca2, cb2) NP_ISSUE(4, y, 0, 1) \
  NP_W15 NP_ADD4(A, z) NP_ISSUE(5, z, 2, 3) \
  NP_W15 NP_ADD4(A, x) CHECK NP_MASKS(ca3, cb3) NP_ISSUE(6, x, 0, 1) \
  NP_W15 NP_ADD4(A, y) NP_ISSUE(7, y, 2, 3) \
  NP_W15 NP_ADD4(A, z) NP_MASKS(ca4, cb4) NP_ISSUE(8, z, 0, 1) \
  NP_W15 NP_ADD4(A, x) NP_ISSUE(9, x, 2, 3) \
  NP_W15 NP_ADD4(A, y) CHECK NP_MASKS(ca5, cb5) NP_ISSUE(10, y, 0, 1) \
  NP_W15 NP_ADD4(A, z) NP_ISSUE(11, z, 2, 3) \
  NP_W15 NP_ADD4(A, x) NP_MASKS(ca6, cb6) NP_ISSUE(12, x, 0, 1) \
  NP_W15 NP_ADD4(A, y) NP_ISSUE(13, y, 2, 3) \
  NP_W15 NP_ADD4(A, z) CHECK NP_MASKS(ca7, cb7) NP_ISSUE(14, z, 0, 1) \
  NP_W15 NP_ADD4(A, x) NP_ISSUE(15, x, 2, 3) \
  NP_W15 NP_ADD4(A, y) \
  NP_W8 NP_ADD4(A, z) \
  NP_W0 NP_ADD4(A, x) \
  ".Lstep_done%=:\n\t" NP_W0

#define NP_OUTPUTS                                                                                              \
  [accA] "+v"(acc_a), [accB] "+v"(acc_b), [aa0] "+v"(aa[0]), [aa1] "+v"(aa[1]), [aa2] "+v"(aa[2]),             \
    [aa3] "+v"(aa[3]), [ab0] "+v"(ab[0]), [ab1] "+v"(ab[1]), [ab2] "+v"(ab[2]), [ab3] "+v"(ab[3]),             \
    [xa0] "=&v"(xa[0]), [xa1] "=&v"(xa[1]), [xa2] "=&v"(xa[2]), [xa3] "=&v"(xa[3]), [xb0] "=&v"(xb[0]),        \
    [xb1] "=&v"(xb[1]), [xb2] "=&v"(xb[2]), [xb3] "=&v"(xb[3]), [ya0] "=&v"(ya[0]), [ya1] "=&v"(ya[1]),        \
    [ya2] "=&v"(ya[2]), [ya3] "=&v"(ya[3]), [yb0] "=&v"(yb[0]), [yb1] "=&v"(yb[1]), [yb2] "=&v"(yb[2]),        \
    [yb3] "=&v"(yb[3]), [za0] "=&v"(za[0]), [za1] "=&v"(za[1]), [za2] "=&v"(za[2]), [za3] "=&v"(za[3]),        \
    [zb0] "=&v"(zb[0]), [zb1] "=&v"(zb[1]), [zb2] "=&v"(zb[2]), [zb3] "=&v"(zb[3]), [evA] "=&v"(evA),          \
    [odA] "=&v"(odA), [evB] "=&v"(evB), [odB] "=&v"(odB), [chkA] "=&v"(chkA), [chkB] "=&v"(chkB),              \
    [tmpA] "=&s"(tmpA), [tmpB] "=&s"(tmpB)
#define NP_INPUTS                                                                                               \
  [one_u] "v"(one_u), [one] "v"(one), [stop] "s"(stop), [validA] "s"(valid_a), [validB] "s"(valid_b),          \
    [ca0] "v"(a[0].x), [ca1] "v"(a[0].y), [ca2] "v"(a[0].z), [ca3] "v"(a[0].w), [ca4] "v"(a[1].x),             \
    [ca5] "v"(a[1].y), [ca6] "v"(a[1].z), [ca7] "v"(a[1].w), [cb0] "v"(b[0].x), [cb1] "v"(b[0].y),             \
    [cb2] "v"(b[0].z), [cb3] "v"(b[0].w), [cb4] "v"(b[1].x), [cb5] "v"(b[1].y), [cb6] "v"(b[1].z),             \
    [cb7] "v"(b[1].w)

/** acc_a, acc_b (sums of rows A and B: binary16 numbers in the low halves, or the bits of floats)
 *  plus the entries that the codes of one step select, in subspace order.  a / b: the step's two
 *  chunks of rows A and B; aa / ab: address registers holding the address of the step's part of
 *  the table in their upper three bytes (the routine writes their lowest bytes only).  CHECK: the
 *  step ends after 8, 16, 32 or 48 subspaces when no row of valid_a / valid_b has a sum whose bits
 *  (as a float's) are at most `stop`. */
template <bool HALF, bool CHECK>
__device__ __forceinline__ void nibble_pack_step(uint32_t& acc_a, uint32_t& acc_b, const u32x4 (&a)[2],
                                                 const u32x4 (&b)[2], uint32_t (&aa)[4], uint32_t (&ab)[4],
                                                 uint32_t one_u, float one, uint32_t stop,
                                                 unsigned long long valid_a, unsigned long long valid_b)
{
  uint32_t xa[4], xb[4], ya[4], yb[4], za[4], zb[4], evA, odA, evB, odB, chkA, chkB;
  unsigned long long tmpA, tmpB;
#define NP_EMIT(ADD1, CHK)                                                                                      \
  asm volatile(NP_BODY(ADD1, CHK)                                                                               \
               : NP_OUTPUTS                                                                                     \
               : NP_INPUTS                                                                                      \
               : "vcc", "scc", "memory")
  if constexpr (HALF && CHECK) {
    NP_EMIT(NP_ADD_H, NP_CHECK_H);
  } else if constexpr (HALF) {
    NP_EMIT(NP_ADD_H, NP_NO_CHECK);
  } else if constexpr (CHECK) {
    NP_EMIT(NP_ADD_F, NP_CHECK_F);
  } else {
    NP_EMIT(NP_ADD_F, NP_NO_CHECK);
  }
#undef NP_EMIT
}

/** decode(encode(score)) as binary16, for the table type chosen at run time.  For fp32 sums an
 *  8-bit entry is decoded as a float, whose top binade binary16 does not reach: the table holds
 *  half of it (exact: a power of two) and the add multiplies by two. */
template <bool IP, bool HALF>
__device__ __forceinline__ _Float16 pack_entry(float score, int lut_dtype)
{
  if (lut_dtype == CUDA_R_8U) {
    using traits = lut_traits<IP ? LUT_FP8S : LUT_FP8U>;
    if constexpr (!HALF) { return _Float16(traits::to_float(traits::encode(score)) * 0.5f); }
    return traits::to_half(traits::encode(score));
  }
  using traits = lut_traits<LUT_F16>;
  return traits::to_half(traits::encode(score));
}

template <bool IP, int PQ_LEN, int NOWN, bool HALF>  // NOWN = pq_dim / 64: subspaces a builder thread owns
__global__ __launch_bounds__(kPackThreads) void scan_nibble_pack_kernel(scan_args a, uint32_t pairs_per_it)
{
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = uint32_t(__builtin_amdgcn_readfirstlane(int(tid >> 6)));
  const uint32_t n_pairs =
    uint32_t(__builtin_amdgcn_readfirstlane(int(a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs)));
  const uint32_t G        = pairs_per_it;
  const uint32_t n_groups = (n_pairs + G - 1u) / G;
  const uint32_t grid     = gridDim.x;
  // Workgroups go to the XCDs in turn; the blocks of one XCD take a contiguous run of pairs.
  const uint32_t lb = (grid & 7u) == 0u ? (blockIdx.x & 7u) * (grid >> 3) + (blockIdx.x >> 3) : blockIdx.x;
  if (lb >= n_groups) { return; }  // whole block, before any barrier
  const uint32_t n_it = (n_groups - lb + grid - 1u) / grid;

  const uint32_t rot         = a.rot_dim;
  const uint32_t nch         = a.pq_dim >> 5;  // 16-byte chunks per row
  const uint32_t n_steps     = nch >> 1;       // steps of 64 subspaces (an even number for inner products)
  const uint32_t table_bytes = a.pq_dim * 32u;

  /* ---- builder state: entry e of subspaces sg, sg + 64, ... ---- */
  const uint32_t e  = tid & 15u;
  const uint32_t sg = tid >> 4;
  float book[NOWN][PQ_LEN];
  if (!a.per_cluster) {
#pragma unroll
    for (int i = 0; i < NOWN; i++) {
#pragma unroll
      for (int t = 0; t < PQ_LEN; t++) {
        book[i][t] = a.pq_centers[(uint64_t(sg + 64u * uint32_t(i)) * PQ_LEN + t) * 16u + e];
      }
    }
  }

  /* ---- scanner state ---- */
  auto* my_cand = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(kPackCandBase)) + wid * kPackWaveCap;
  uint32_t one_u = 1u;
  asm volatile("" : "+v"(one_u));
  float one = a.lut_dtype == CUDA_R_8U ? 2.0f : 1.0f;  // factor of the entries (fp32 sums)
  asm volatile("" : "+v"(one));
  // a sum as a float: the binary16 number in the low half, or the register's bits
  auto sum_of = [](uint32_t acc) {
    return HALF ? float(__builtin_bit_cast(_Float16, uint16_t(acc))) : __uint_as_float(acc);
  };

  for (uint32_t it = 0; it < n_it; it++) {
    const uint32_t first = (lb + it * grid) * G;  // first pair of the iteration

    // the scanner wave's pair: its record and the query's bound are on their way during the build
    const bool scanner = wid < G && first + wid < n_pairs;
    pair_desc my_d{};
    uint32_t pre_thr = 0xFFFFFFFFu;
    if (scanner) {
      my_d = a.desc[first + wid];
      if (my_d.n_rows != 0) { pre_thr = a.query_kth[my_d.q]; }
    }

    /* ---- tables of the iteration's pairs: every wave builds ---- */
    {
      // lane g holds the record of the iteration's pair g: no table waits for a record of its own
      uint32_t rec_q = 0, rec_label = 0, rec_rows = 0;
      if (first + lane < n_pairs && lane < G) {
        const pair_desc* rec = a.desc + (first + lane);
        rec_q                = rec->q;
        rec_label            = rec->label;
        rec_rows             = rec->n_rows;
      }
      for (uint32_t g = 0; g < G; g++) {
        if (__builtin_amdgcn_readlane(int(rec_rows), int(g)) == 0) { continue; }  // uniform: no pair, or an empty list
        const uint32_t q     = uint32_t(__builtin_amdgcn_readlane(int(rec_q), int(g)));
        const uint32_t label = uint32_t(__builtin_amdgcn_readlane(int(rec_label), int(g)));
        // the thread's terms: subspace sg + 64 i at a fixed distance from subspace sg
        const float* qp = a.rot_q + uint64_t(q) * rot + sg * uint32_t(PQ_LEN);
        const float* cp = a.centers_rot + uint64_t(label) * rot + sg * uint32_t(PQ_LEN);
        typedef float term_vec __attribute__((ext_vector_type(PQ_LEN)));
        term_vec qs[NOWN], cs[NOWN];
#pragma unroll
        for (int i = 0; i < NOWN; i++) {
          qs[i] = *reinterpret_cast<const term_vec*>(qp + i * 64 * PQ_LEN);
          cs[i] = *reinterpret_cast<const term_vec*>(cp + i * 64 * PQ_LEN);
        }
        float cb[PQ_LEN];
        if (a.per_cluster) {
#pragma unroll
          for (int d = 0; d < PQ_LEN; d++) { cb[d] = a.pq_centers[(uint64_t(label) * PQ_LEN + d) * 16u + e]; }
        }
        // entry (subspace, e) at table + subspace * 32 + e * 2
        auto* mine = reinterpret_cast<LDS_AS _Float16*>(uintptr_t(kPackTableBase + g * table_bytes + (sg * 16u + e) * 2u));
#pragma unroll
        for (int i = 0; i < NOWN; i++) {
          float score = 0.0f;
#pragma unroll
          for (int d = 0; d < PQ_LEN; d++) {
            const float qd = qs[i][d];
            const float cd = cs[i][d];
            const float pqc = a.per_cluster ? cb[d] : book[i][d];
            if constexpr (!IP) {
              float diff = qd - cd;
              diff -= pqc;
              score = fmaf(diff, diff, score);
            } else {
              // the rounded product, as the reference subtracts it: kept out of the compiler's sight, which
              // would fuse the multiplication into the subtraction (one rounding instead of two)
              float cq = cd * qd;
              asm volatile("" : "+v"(cq));
              score -= cq;
              score = fmaf(-qd, pqc, score);
            }
          }
          mine[i * 64 * 16] = pack_entry<IP, HALF>(score, a.lut_dtype);
        }
      }
    }
    __syncthreads();

    /* ---- scan: wave w takes pair w ---- */
    if (scanner) {
      const uint32_t n_rows     = my_d.n_rows;
      const uint32_t sample_off = my_d.sample_off;
      unsigned long long* out   = a.out_keys + uint64_t(my_d.slot) * a.k;
      uint32_t wcount           = 0;
      if (n_rows != 0) {
        const uint8_t* list_data = my_d.data;
        const int64_t* list_ids  = a.filter_bits != nullptr ? a.inds_ptrs[my_d.label] : nullptr;
        const bool cosine        = a.metric == int(DistanceType::CosineExpanded);
        // the wave's bound: a key, and the same as a score (no bound: +inf; NaN scores never pass)
        uint32_t thr = uint32_t(__builtin_amdgcn_readfirstlane(int(pre_thr)));
        float thr_f  = thr >= 0xFF800000u ? __uint_as_float(0x7F800000u) : unorder_f32(thr);
        const uint32_t table = kPackTableBase + wid * table_bytes;
        uint32_t aa[4], ab[4];

        // chunks 2 * step, 2 * step + 1 of a row
        auto load_step = [&](uint32_t row, uint32_t step, u32x4 (&dst)[2]) {
          const uintptr_t p = reinterpret_cast<uintptr_t>(list_data) + uint64_t(row >> 5) * (uint64_t(nch) * 512u) +
                              uint64_t(row & 31u) * 16u + uint64_t(step) * 1024u;
          dst[0] = *reinterpret_cast<const GLOBAL_AS u32x4*>(p);
          dst[1] = *reinterpret_cast<const GLOBAL_AS u32x4*>(p + 512u);
        };
        auto in_play = [&](uint32_t row) {
          bool valid = row < n_rows;
          if (list_ids != nullptr) {
            if (valid) {
              const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[row];
              valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
            }
          }
          return valid;
        };
        // the rows whose scores pass the bound join the wave's candidates
        auto take = [&](float score, bool valid, uint32_t row) {
          const unsigned long long mask = __builtin_amdgcn_ballot_w64(valid && score <= thr_f);
          if (mask == 0ull) { return; }
          if (wcount + 64u > kPackWaveCap) {
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
          if (pass) { my_cand[wcount + below] = (static_cast<unsigned long long>(okey) << 32) | (sample_off + row); }
          wcount += uint32_t(__popcll(mask2));
        };

        const uint32_t n_tiles = (n_rows + 127u) >> 7;  // of 128 rows: two per lane
        u32x4 cur_a[2], cur_b[2], nxt_a[2], nxt_b[2];
        load_step(lane < n_rows ? lane : 0u, 0u, cur_a);
        load_step(lane + 64u < n_rows ? lane + 64u : 0u, 0u, cur_b);
        if constexpr (!IP) {
          // L2: most tiles end inside their first step (no row can still win), so what is worth having
          // on its way is the next tile's first step, not this tile's next one.  The two buffers
          // swap roles from tile to tile; a tile whose rows stay in play fetches its later steps
          // when it gets there.
          auto l2_tile = [&](uint32_t tile, u32x4 (&pa)[2], u32x4 (&pb)[2], u32x4 (&qa)[2], u32x4 (&qb)[2]) {
            const uint32_t row_a = tile * 128u + lane;
            const uint32_t row_b = row_a + 64u;
            const bool valid_a   = in_play(row_a);
            const bool valid_b   = in_play(row_b);
            {
              // requested without a condition (past the end: row 0 again)
              const uint32_t na = row_a + 128u, nb = row_b + 128u;
              load_step(na < n_rows ? na : 0u, 0u, qa);
              load_step(nb < n_rows ? nb : 0u, 0u, qb);
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
              aa[i] = table;
              ab[i] = table;
              asm volatile("" : "+v"(aa[i]), "+v"(ab[i]));
            }
            uint32_t acc_a = 0, acc_b = 0;  // zeros of either type
            // inside a step the bound is compared as bits (sums are not negative: past the bound =
            // past its bits); between steps as numbers
            const uint32_t stop_bits        = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
            const unsigned long long mask_a = __builtin_amdgcn_ballot_w64(valid_a);
            const unsigned long long mask_b = __builtin_amdgcn_ballot_w64(valid_b);
            auto all_past = [&]() {
              return __builtin_amdgcn_ballot_w64((valid_a && !(sum_of(acc_a) > thr_f)) ||
                                                 (valid_b && !(sum_of(acc_b) > thr_f))) == 0ull;
            };
            nibble_pack_step<HALF, true>(acc_a, acc_b, pa, pb, aa, ab, one_u, one, stop_bits, mask_a, mask_b);
            bool stopped = all_past();
            for (uint32_t step = 1; step < n_steps && !stopped; step++) {
              load_step(row_a < n_rows ? row_a : 0u, step, pa);
              load_step(row_b < n_rows ? row_b : 0u, step, pb);
#pragma unroll
              for (int i = 0; i < 4; i++) {
                aa[i] += kPackStepBytes;
                ab[i] += kPackStepBytes;
              }
              nibble_pack_step<HALF, true>(acc_a, acc_b, pa, pb, aa, ab, one_u, one, stop_bits, mask_a, mask_b);
              stopped = step + 1u < n_steps && all_past();
            }
            if (stopped) { return; }  // every row in play is past the bound
            take(sum_of(acc_a), valid_a, row_a);
            take(sum_of(acc_b), valid_b, row_b);
          };
          if (a.rare_exits == 0 || (n_steps & 1u) != 0u) {
            for (uint32_t tile = 0; tile < n_tiles; tile += 2u) {
              l2_tile(tile, cur_a, cur_b, nxt_a, nxt_b);
              if (tile + 1u < n_tiles) { l2_tile(tile + 1u, nxt_a, nxt_b, cur_a, cur_b); }
            }
          } else {
            // Pairs whose rows mostly stay under the bound (no bound yet, or the survivors of the
            // screen): a tile's next step is what should be on its way, as for inner products, and a
            // tile that does end early fetches the next one's first step afresh.
            for (uint32_t tile = 0; tile < n_tiles; tile++) {
              const uint32_t row_a = tile * 128u + lane;
              const uint32_t row_b = row_a + 64u;
              const bool valid_a   = in_play(row_a);
              const bool valid_b   = in_play(row_b);
#pragma unroll
              for (int i = 0; i < 4; i++) {
                aa[i] = table;
                ab[i] = table;
                asm volatile("" : "+v"(aa[i]), "+v"(ab[i]));
              }
              uint32_t acc_a = 0, acc_b = 0;
              bool stopped   = false;
              const uint32_t stop_bits        = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
              const unsigned long long mask_a = __builtin_amdgcn_ballot_w64(valid_a);
              const unsigned long long mask_b = __builtin_amdgcn_ballot_w64(valid_b);
              auto all_past = [&]() {
                return __builtin_amdgcn_ballot_w64((valid_a && !(sum_of(acc_a) > thr_f)) ||
                                                   (valid_b && !(sum_of(acc_b) > thr_f))) == 0ull;
              };
              for (uint32_t step = 0; step < n_steps; step += 2) {
                {
                  const uint32_t ra = row_a < n_rows ? row_a : 0u;
                  const uint32_t rb = row_b < n_rows ? row_b : 0u;
                  load_step(ra, step + 1u, nxt_a);
                  load_step(rb, step + 1u, nxt_b);
                }
                nibble_pack_step<HALF, true>(acc_a, acc_b, cur_a, cur_b, aa, ab, one_u, one, stop_bits, mask_a, mask_b);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                  aa[i] += kPackStepBytes;
                  ab[i] += kPackStepBytes;
                }
                if (all_past()) {
                  stopped = true;
                  break;
                }
                {
                  const bool more   = step + 2u < n_steps;
                  const uint32_t na = more ? row_a : row_a + 128u;
                  const uint32_t nb = more ? row_b : row_b + 128u;
                  load_step(na < n_rows ? na : 0u, more ? step + 2u : 0u, cur_a);
                  load_step(nb < n_rows ? nb : 0u, more ? step + 2u : 0u, cur_b);
                }
                nibble_pack_step<HALF, true>(acc_a, acc_b, nxt_a, nxt_b, aa, ab, one_u, one, stop_bits, mask_a, mask_b);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                  aa[i] += kPackStepBytes;
                  ab[i] += kPackStepBytes;
                }
                if (step + 2u < n_steps && all_past()) {
                  stopped = true;
                  break;
                }
              }
              if (stopped) {
                // the codes on their way are of this tile: the next tile's first step is fetched afresh
                if (tile + 1u < n_tiles) {
                  const uint32_t na = row_a + 128u, nb = row_b + 128u;
                  load_step(na < n_rows ? na : 0u, 0u, cur_a);
                  load_step(nb < n_rows ? nb : 0u, 0u, cur_b);
                }
                continue;  // every row in play is past the bound
              }
              take(sum_of(acc_a), valid_a, row_a);
              take(sum_of(acc_b), valid_b, row_b);
            }
          }
        } else {
          for (uint32_t tile = 0; tile < n_tiles; tile++) {
            const uint32_t row_a = tile * 128u + lane;
            const uint32_t row_b = row_a + 64u;
            const bool valid_a   = in_play(row_a);
            const bool valid_b   = in_play(row_b);
  #pragma unroll
            for (int i = 0; i < 4; i++) {
              aa[i] = table;
              ab[i] = table;
              asm volatile("" : "+v"(aa[i]), "+v"(ab[i]));
            }
            uint32_t acc_a = 0, acc_b = 0;  // zeros of either type
            for (uint32_t step = 0; step < n_steps; step += 2) {
              // the step after this one: of the same rows, or the first of the next tile's (past the
              // end: row 0 again); requested without a condition
              {
                const uint32_t ra = row_a < n_rows ? row_a : 0u;
                const uint32_t rb = row_b < n_rows ? row_b : 0u;
                load_step(ra, step + 1u, nxt_a);
                load_step(rb, step + 1u, nxt_b);
              }
              nibble_pack_step<HALF, false>(acc_a, acc_b, cur_a, cur_b, aa, ab, one_u, one, 0u, 0ull, 0ull);
  #pragma unroll
              for (int i = 0; i < 4; i++) {
                aa[i] += kPackStepBytes;
                ab[i] += kPackStepBytes;
              }
              {
                const bool more   = step + 2u < n_steps;
                const uint32_t na = more ? row_a : row_a + 128u;
                const uint32_t nb = more ? row_b : row_b + 128u;
                load_step(na < n_rows ? na : 0u, more ? step + 2u : 0u, cur_a);
                load_step(nb < n_rows ? nb : 0u, more ? step + 2u : 0u, cur_b);
              }
              nibble_pack_step<HALF, false>(acc_a, acc_b, nxt_a, nxt_b, aa, ab, one_u, one, 0u, 0ull, 0ull);
  #pragma unroll
              for (int i = 0; i < 4; i++) {
                aa[i] += kPackStepBytes;
                ab[i] += kPackStepBytes;
              }
            }
            if constexpr (HALF) {
              _Float16 ha = __builtin_bit_cast(_Float16, uint16_t(acc_a));
              _Float16 hb = __builtin_bit_cast(_Float16, uint16_t(acc_b));
              if (cosine) {
                ha = _Float16(ha + _Float16(1));
                hb = _Float16(hb + _Float16(1));
              }
              take(float(ha), valid_a, row_a);
              take(float(hb), valid_b, row_b);
            } else {
              float fa = __uint_as_float(acc_a);
              float fb = __uint_as_float(acc_b);
              if (cosine) {
                fa += 1.0f;
                fb += 1.0f;
              }
              take(fa, valid_a, row_a);
              take(fb, valid_b, row_b);
            }
          }
        }
        if (wcount >= a.k) {
          const uint32_t kth = wcount <= 64u ? wave_select_keys<1>(my_cand, lane, wcount, a.k)
                                             : wave_select_keys<2>(my_cand, lane, wcount, a.k);
          wcount = a.k;
          if (lane == 0) { atomicMin(&a.query_kth[my_d.q], kth); }
        }
      }
      for (uint32_t t = lane; t < a.k; t += 64u) { out[t] = t < wcount ? my_cand[t] : kInvalidKey; }
    }
    __syncthreads();  // the tables are free again
  }
}

uint32_t pack_pairs_per_iteration(const scan_args& a)
{
  const uint32_t fit = (kPackLdsBytes - kPackTableBase) / (a.pq_dim * 32u);
  return fit < kPackMaxPairs ? fit : kPackMaxPairs;
}

template <bool IP, int PQ_LEN, int NOWN, bool HALF>
void launch_pack_sums(const scan_args& a, hipStream_t stream)
{
  auto kernel = scan_nibble_pack_kernel<IP, PQ_LEN, NOWN, HALF>;
  // per instance: the whole LDS of a CU belongs to the one resident block
  static const int attr_set = [&] {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, int(kPackLdsBytes)));
    return 1;
  }();
  (void)attr_set;
  const uint32_t G = pack_pairs_per_iteration(a);
  uint32_t grid    = uint32_t(device_cu_count());
  if (a.n_pairs_dev == nullptr) {
    const uint32_t n_groups = (a.n_pairs + G - 1u) / G;
    if (grid > n_groups) { grid = n_groups; }
    if (grid == 0) { return; }
  }
  kernel<<<grid, kPackThreads, kPackTableBase + G * a.pq_dim * 32u, stream>>>(a, G);
  CUVS_HIP_TRY(hipGetLastError());
}

template <bool IP, int PQ_LEN, int NOWN>
void launch_pack_instance(const scan_args& a, hipStream_t stream)
{
  if (a.out_half) {
    launch_pack_sums<IP, PQ_LEN, NOWN, true>(a, stream);
  } else {
    launch_pack_sums<IP, PQ_LEN, NOWN, false>(a, stream);
  }
}

template <bool IP, int PQ_LEN>
void launch_pack_width(const scan_args& a, hipStream_t stream)
{
  switch (a.pq_dim >> 6) {
    case 2: launch_pack_instance<IP, PQ_LEN, 2>(a, stream); break;
    case 4: launch_pack_instance<IP, PQ_LEN, 4>(a, stream); break;
    case 6: launch_pack_instance<IP, PQ_LEN, 6>(a, stream); break;
    case 8: launch_pack_instance<IP, PQ_LEN, 8>(a, stream); break;
    default:
      // an odd number of steps: the L2 tile loop takes them one by one
      if constexpr (!IP) {
        switch (a.pq_dim >> 6) {
          case 1: launch_pack_instance<IP, PQ_LEN, 1>(a, stream); break;
          case 3: launch_pack_instance<IP, PQ_LEN, 3>(a, stream); break;
          case 5: launch_pack_instance<IP, PQ_LEN, 5>(a, stream); break;
          case 7: launch_pack_instance<IP, PQ_LEN, 7>(a, stream); break;
          default: break;
        }
      }
      break;
  }
}

template <bool IP>
void launch_pack_len(const scan_args& a, hipStream_t stream)
{
  if (a.pq_len == 1) { launch_pack_width<IP, 1>(a, stream); }
  if (a.pq_len == 2) { launch_pack_width<IP, 2>(a, stream); }
  if (a.pq_len == 4) { launch_pack_width<IP, 4>(a, stream); }
}

}  // namespace

bool scan_nibble_pack_supported(const scan_args& a)
{
  if (!a.fused || a.pq_bits != 4 || a.k > kPackMaxK) { return false; }
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  // steps of 64 subspaces: in pairs for inner products (one step's codes arrive while the other's are summed)
  if (a.pq_dim % (ip ? 128u : 64u) != 0 || a.pq_dim > 512u || a.rot_dim != a.pq_dim * a.pq_len) { return false; }
  if (a.pq_len != 1 && a.pq_len != 2 && a.pq_len != 4) { return false; }
  return a.lut_dtype == CUDA_R_16F || a.lut_dtype == CUDA_R_8U;
}

bool launch_scan_nibble_pack(const scan_args& a, hipStream_t stream)
{
  if (!scan_nibble_pack_supported(a) || a.n_queries == 0 || a.desc == nullptr) { return false; }
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (ip) {
    launch_pack_len<true>(a, stream);
  } else {
    launch_pack_len<false>(a, stream);
  }
  return true;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
