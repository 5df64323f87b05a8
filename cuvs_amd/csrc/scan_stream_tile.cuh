/*
 * What the CU-wide scan kernels for 8-bit codes share (scan_stream.hip: a pair's whole table in LDS;
 * scan_slab.hip: the table in slabs of 64 subspaces): the form of a table entry, and the sum of a
 * tile's table entries as one block of assembly.
 */
#pragma once

#include "scan_wave_select.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte chunk of codes
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void block_barrier()
{
  // LDS traffic of this wave is complete; global loads stay in flight across the barrier
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

/** `v` in a register the compiler knows nothing about (it would otherwise fold a multiplication by
 *  one away and lose the single-instruction widening multiply-add). */
__device__ __forceinline__ float opaque_float(float v)
{
  asm volatile("" : "+v"(v));
  return v;
}

/** The 16 bits stored for a table entry: a binary16 number in the form the scan adds - the entry
 *  itself for fp16 tables; for 8-bit tables the decoded value decode(encode(score)), which the
 *  reference computes again at every lookup, as it is when the sums are binary16, and halved when
 *  they are fp32 (half of every decoded 8-bit value is a binary16 number, the largest ones
 *  themselves are not), the scan then adding twice the entry, which is exact. */
template <int LUT, bool OUT_HALF>
__device__ __forceinline__ uint16_t table_entry(float score)
{
  using traits = lut_traits<LUT>;
  const auto e = traits::encode(score);
  if constexpr (LUT == LUT_F16) {
    return __builtin_bit_cast(uint16_t, e);
  } else if constexpr (OUT_HALF) {
    return __builtin_bit_cast(uint16_t, traits::to_half(e));
  } else {
    // 2^-16 * 1.0625 .. 63488, four significant bits: exact in binary16 (subnormal at the low end)
    return __builtin_bit_cast(uint16_t, _Float16(traits::to_float(e) * 0.5f));
  }
}

/* ---- One tile of 64 rows, as a single block of assembly.  The compiler would extract each code
 * byte, form a full address and wait for every read; and a lookup whose register is written some
 * hundred cycles after the read was issued cannot be left to it piecewise (it treats the register as
 * holding its value from the instruction that issued the read on, and may copy it at a branch).
 *
 * A lookup is two vector instructions: one sub-dword shift puts 2 * code into the low half of an
 * address register whose high half holds the table's 64 KB window (the subspace's offset sits in
 * the read's immediate field), and the entry that ds_read_u16 returns is added.  The lookups go in
 * groups of eight (two code dwords); two groups are in flight while a third is added, so a wave
 * always has reads queued.  After each chunk of sixteen subspaces but the last, an L2 scan ends the
 * tile if no row in play can still beat the bound (sums only grow; early stop of compute_score in
 * the reference): the group that is in flight then is awaited and dropped. ---- */
#define ST_SDWA(a, c, sel)                                                                                   \
  "v_lshlrev_b32_sdwa %[" #a "], %[one_u], %[" #c "] dst_sel:WORD_0 dst_unused:UNUSED_PRESERVE src0_sel:DWORD " \
  "src1_sel:BYTE_" #sel "\n\t"
/* the read of subspace 8 o + i: 16-bit entries 512 bytes a subspace, or (RD32) fp32 entries 1 KB a subspace */
#define ST_RD16(v, a, o, i) "ds_read_u16 %[" #v "], %[" #a "] offset:%[immg]+" #o "*4096+" #i "*512\n\t"
#define ST_RD32(v, a, o, i) "ds_read_b32 %[" #v "], %[" #a "] offset:%[immg]+" #o "*8192+" #i "*1024\n\t"
/* (RD8) one-byte entries, 256 bytes a subspace: the 8-bit code of an unsigned 8-bit table entry */
#define ST_RD8(v, a, o, i) "ds_read_u8 %[" #v "], %[" #a "] offset:%[immg]+" #o "*2048+" #i "*256\n\t"
/* group o: subspaces 8 o .. 8 o + 7, code dwords ca, cb, entries into V0 .. V7 */
#define ST_ISSUE(RD, o, ca, cb, V)                                                                 \
  ST_SDWA(a0, ca, 0) ST_SDWA(a1, ca, 1) ST_SDWA(a2, ca, 2) ST_SDWA(a3, ca, 3)                      \
  ST_SDWA(a4, cb, 0) ST_SDWA(a5, cb, 1) ST_SDWA(a6, cb, 2) ST_SDWA(a7, cb, 3)                      \
  RD(V##0, a0, o, 0) RD(V##1, a1, o, 1) RD(V##2, a2, o, 2) RD(V##3, a3, o, 3)                      \
  RD(V##4, a4, o, 4) RD(V##5, a5, o, 5) RD(V##6, a6, o, 6) RD(V##7, a7, o, 7)
/* the two halves of a group: one code dword each */
#define ST_ISSUE_LO(RD, o, ca, V)                                                                  \
  ST_SDWA(a0, ca, 0) ST_SDWA(a1, ca, 1) ST_SDWA(a2, ca, 2) ST_SDWA(a3, ca, 3)                      \
  RD(V##0, a0, o, 0) RD(V##1, a1, o, 1) RD(V##2, a2, o, 2) RD(V##3, a3, o, 3)
#define ST_ISSUE_HI(RD, o, cb, V)                                                                  \
  ST_SDWA(a4, cb, 0) ST_SDWA(a5, cb, 1) ST_SDWA(a6, cb, 2) ST_SDWA(a7, cb, 3)                      \
  RD(V##4, a4, o, 4) RD(V##5, a5, o, 5) RD(V##6, a6, o, 6) RD(V##7, a7, o, 7)
#define ST_WAIT4 "s_waitcnt lgkmcnt(4)\n\t"
#define ST_WAIT8 "s_waitcnt lgkmcnt(8)\n\t"
#define ST_WAIT0 "s_waitcnt lgkmcnt(0)\n\t"
/* fp32 sums: entry * scale + sum in one instruction that widens the binary16 entry (exact product) */
#define ST_ADD_F32_1(v) "v_fma_mix_f32 %[acc], %[" #v "], %[one], %[acc] op_sel_hi:[1,0,0]\n\t"
#define ST_ADD_F16_1(v) "v_add_f16_e32 %[acc], %[acc], %[" #v "]\n\t"
/* fp32 entries */
#define ST_ADD_W32_1(v) "v_add_f32_e32 %[acc], %[acc], %[" #v "]\n\t"
/* one-byte entries e of an unsigned 8-bit table: decoded in the register, as the fp32 number with
 * the bits (e << 20) + 0x38080000 (`one` holds that constant) or the binary16 number with the bits
 * (e << 7) + 0x40, then added */
#define ST_ADD_B32_1(v) "v_lshl_add_u32 %[" #v "], %[" #v "], 20, %[one]\n\tv_add_f32_e32 %[acc], %[acc], %[" #v "]\n\t"
#define ST_ADD_B16_1(v) "v_lshl_add_u32 %[" #v "], %[" #v "], 7, 64\n\tv_add_f16_e32 %[acc], %[acc], %[" #v "]\n\t"
#define ST_ADD8(ADD1, V) ADD1(V##0) ADD1(V##1) ADD1(V##2) ADD1(V##3) ADD1(V##4) ADD1(V##5) ADD1(V##6) ADD1(V##7)
#define ST_ADD4_LO(ADD1, V) ADD1(V##0) ADD1(V##1) ADD1(V##2) ADD1(V##3)
#define ST_ADD4_HI(ADD1, V) ADD1(V##4) ADD1(V##5) ADD1(V##6) ADD1(V##7)
#define ST_ADD_F32(V) ST_ADD8(ST_ADD_F32_1, V)
#define ST_ADD_F16(V) ST_ADD8(ST_ADD_F16_1, V)
#define ST_ADD_W32(V) ST_ADD8(ST_ADD_W32_1, V)
#define ST_ADD_F32_LO(V) ST_ADD4_LO(ST_ADD_F32_1, V)
#define ST_ADD_F32_HI(V) ST_ADD4_HI(ST_ADD_F32_1, V)
#define ST_ADD_F16_LO(V) ST_ADD4_LO(ST_ADD_F16_1, V)
#define ST_ADD_F16_HI(V) ST_ADD4_HI(ST_ADD_F16_1, V)
#define ST_ADD_W32_LO(V) ST_ADD4_LO(ST_ADD_W32_1, V)
#define ST_ADD_W32_HI(V) ST_ADD4_HI(ST_ADD_W32_1, V)
#define ST_ADD_B32(V) ST_ADD8(ST_ADD_B32_1, V)
#define ST_ADD_B32_LO(V) ST_ADD4_LO(ST_ADD_B32_1, V)
#define ST_ADD_B32_HI(V) ST_ADD4_HI(ST_ADD_B32_1, V)
#define ST_ADD_B16(V) ST_ADD8(ST_ADD_B16_1, V)
#define ST_ADD_B16_LO(V) ST_ADD4_LO(ST_ADD_B16_1, V)
#define ST_ADD_B16_HI(V) ST_ADD4_HI(ST_ADD_B16_1, V)
/* rows in play whose sum is not past the bound; none: leave */
#define ST_CHECK_F32                                 \
  "v_cmp_ge_u32_e32 vcc, %[stop], %[acc]\n\t"        \
  "s_and_b64 %[tmp], vcc, %[valid]\n\t"              \
  "s_cbranch_scc0 .Ltile_done%=\n\t"
#define ST_CHECK_F16                                 \
  "v_cvt_f32_f16_e32 %[chk], %[acc]\n\t"             \
  "v_cmp_ge_u32_e32 vcc, %[stop], %[chk]\n\t"        \
  "s_and_b64 %[tmp], vcc, %[valid]\n\t"              \
  "s_cbranch_scc0 .Ltile_done%=\n\t"
#define ST_NO_CHECK ""
/* The first chunk starts with half as many lookups in flight and looks at the bound after four
 * subspaces already: most tiles that cannot win are known by then, and leave with eight lookups
 * issued.  The sum starts from the value the caller put into the accumulator.  The waits count
 * this block's own reads: nothing else that counts on lgkmcnt and may complete out of order (a
 * scalar load) may be in flight when the block starts. */
#define ST_FIRST(RD, ADD, CHECK)                                                \
  ST_ISSUE_LO(RD, 0, c0, va) ST_ISSUE_HI(RD, 0, c1, va)                         \
  ST_WAIT4 ADD##_LO(va) CHECK ST_ISSUE(RD, 1, c2, c3, vb)                       \
  ST_WAIT8 ADD##_HI(va) CHECK ST_ISSUE(RD, 2, c4, c5, va)                       \
  ST_WAIT8 ADD(vb) CHECK ST_ISSUE(RD, 3, c6, c7, vb)
/* a chunk that is not the last: its two groups are added, groups o + 2 and o + 3 issued */
#define ST_CHUNK(RD, o0, o1, o2, o3, c4, c5, c6, c7, ADD, CHECK)  \
  ST_WAIT8 ADD(va) CHECK ST_ISSUE(RD, o2, c4, c5, va)             \
  ST_WAIT8 ADD(vb) CHECK ST_ISSUE(RD, o3, c6, c7, vb)
#define ST_TAIL(ADD) ST_WAIT8 ADD(va) ST_WAIT0 ADD(vb) ".Ltile_done%=:\n\t" ST_WAIT0
#define ST_BODY_2(RD, ADD, CHECK) ST_FIRST(RD, ADD, CHECK) ST_TAIL(ADD)
#define ST_BODY_3(RD, ADD, CHECK) \
  ST_FIRST(RD, ADD, CHECK) ST_CHUNK(RD, 2, 3, 4, 5, c8, c9, c10, c11, ADD, CHECK) ST_TAIL(ADD)
#define ST_BODY_4(RD, ADD, CHECK)                                                            \
  ST_FIRST(RD, ADD, CHECK) ST_CHUNK(RD, 2, 3, 4, 5, c8, c9, c10, c11, ADD, CHECK)            \
  ST_CHUNK(RD, 4, 5, 6, 7, c12, c13, c14, c15, ADD, CHECK) ST_TAIL(ADD)

#define ST_OUTPUTS                                                                                              \
  [acc] "+v"(acc), [chk] "=&v"(chk), [tmp] "=&s"(tmp), [a0] "+v"(ad[0]), [a1] "+v"(ad[1]), [a2] "+v"(ad[2]),     \
    [a3] "+v"(ad[3]), [a4] "+v"(ad[4]), [a5] "+v"(ad[5]), [a6] "+v"(ad[6]), [a7] "+v"(ad[7]),                   \
    [va0] "=&v"(va[0]), [va1] "=&v"(va[1]), [va2] "=&v"(va[2]), [va3] "=&v"(va[3]), [va4] "=&v"(va[4]),         \
    [va5] "=&v"(va[5]), [va6] "=&v"(va[6]), [va7] "=&v"(va[7]), [vb0] "=&v"(vb[0]), [vb1] "=&v"(vb[1]),         \
    [vb2] "=&v"(vb[2]), [vb3] "=&v"(vb[3]), [vb4] "=&v"(vb[4]), [vb5] "=&v"(vb[5]), [vb6] "=&v"(vb[6]),         \
    [vb7] "=&v"(vb[7])
#define ST_COMMON_INPUTS \
  [one_u] "v"(one_u), [one] "v"(one), [stop] "s"(stop), [valid] "s"(valid), [immg] "n"(IMMG)
#define ST_CODES_2                                                                                              \
  [c0] "v"(cur[0].x), [c1] "v"(cur[0].y), [c2] "v"(cur[0].z), [c3] "v"(cur[0].w), [c4] "v"(cur[1].x),           \
    [c5] "v"(cur[1].y), [c6] "v"(cur[1].z), [c7] "v"(cur[1].w)
#define ST_CODES_3 \
  ST_CODES_2, [c8] "v"(cur[2].x), [c9] "v"(cur[2].y), [c10] "v"(cur[2].z), [c11] "v"(cur[2].w)
#define ST_CODES_4 \
  ST_CODES_3, [c12] "v"(cur[3].x), [c13] "v"(cur[3].y), [c14] "v"(cur[3].z), [c15] "v"(cur[3].w)

/** `start` plus the table entries of a tile's rows in subspace order, as the bits of a float
 *  (HALF: of a binary16 number in the low half).  `cur` may hold more chunks than the NCH that are
 *  summed.  CHECK: end the tile when no row of `valid` has a sum whose bits are at most `stop`.
 *  IMMG: offset of the table inside its 64 KB window, which the high halves of the address
 *  registers `ad` name (the routine changes their low halves only); `one` is the factor of the
 *  entries (fp32 sums), one_u the integer 1.  WIDE: the table holds fp32 entries, 1 KB a subspace,
 *  added as they are; one_u is then 2 (the shift that turns a code into its entry's offset).
 *  BYTE: the table holds the one-byte codes of an unsigned 8-bit table, 256 bytes a subspace,
 *  decoded after the read; one_u is then 0 and `one` the constant of the fp32 decoding. */
template <int NCH, bool HALF, bool CHECK, int IMMG, bool WIDE = false, bool BYTE = false, int NCUR = NCH>
__device__ __forceinline__ uint32_t stream_tile_sum(const u32x4 (&cur)[NCUR], uint32_t (&ad)[8], uint32_t one_u, float one,
                                                    uint32_t stop, unsigned long long valid, uint32_t start = 0u)
{
  static_assert(NCH >= 2 && NCH <= 4 && NCH <= NCUR, "two to four chunks of sixteen subspaces");
  static_assert(IMMG >= 0 && IMMG + (NCH * 16 - 1) * (WIDE ? 1024 : 512) < 65536, "the read's offset field has 16 bits");
  static_assert(!(WIDE && HALF), "fp32 entries are summed in fp32");
  static_assert(!(WIDE && BYTE), "one entry size");
  uint32_t acc = start, chk, va[8], vb[8];
  unsigned long long tmp;
#define ST_EMIT(BODY, RD, ADD, CHK, ...) \
  asm volatile(BODY(RD, ADD, CHK) : ST_OUTPUTS : ST_COMMON_INPUTS, __VA_ARGS__ : "vcc", "scc", "memory")
#define ST_EMIT_KIND(BODY, ...)                                              \
  if constexpr (BYTE && !HALF && CHECK) {                                    \
    ST_EMIT(BODY, ST_RD8, ST_ADD_B32, ST_CHECK_F32, __VA_ARGS__);            \
  } else if constexpr (BYTE && !HALF && !CHECK) {                            \
    ST_EMIT(BODY, ST_RD8, ST_ADD_B32, ST_NO_CHECK, __VA_ARGS__);             \
  } else if constexpr (BYTE && HALF && CHECK) {                              \
    ST_EMIT(BODY, ST_RD8, ST_ADD_B16, ST_CHECK_F16, __VA_ARGS__);            \
  } else if constexpr (BYTE && HALF && !CHECK) {                             \
    ST_EMIT(BODY, ST_RD8, ST_ADD_B16, ST_NO_CHECK, __VA_ARGS__);             \
  } else if constexpr (WIDE && CHECK) {                                      \
    ST_EMIT(BODY, ST_RD32, ST_ADD_W32, ST_CHECK_F32, __VA_ARGS__);           \
  } else if constexpr (WIDE && !CHECK) {                                     \
    ST_EMIT(BODY, ST_RD32, ST_ADD_W32, ST_NO_CHECK, __VA_ARGS__);            \
  } else if constexpr (!HALF && CHECK) {                                     \
    ST_EMIT(BODY, ST_RD16, ST_ADD_F32, ST_CHECK_F32, __VA_ARGS__);           \
  } else if constexpr (!HALF && !CHECK) {                                    \
    ST_EMIT(BODY, ST_RD16, ST_ADD_F32, ST_NO_CHECK, __VA_ARGS__);            \
  } else if constexpr (HALF && CHECK) {                                      \
    ST_EMIT(BODY, ST_RD16, ST_ADD_F16, ST_CHECK_F16, __VA_ARGS__);           \
  } else {                                                                   \
    ST_EMIT(BODY, ST_RD16, ST_ADD_F16, ST_NO_CHECK, __VA_ARGS__);            \
  }
  if constexpr (NCH == 2) {
    ST_EMIT_KIND(ST_BODY_2, ST_CODES_2)
  } else if constexpr (NCH == 3) {
    ST_EMIT_KIND(ST_BODY_3, ST_CODES_3)
  } else {
    ST_EMIT_KIND(ST_BODY_4, ST_CODES_4)
  }
#undef ST_EMIT_KIND
#undef ST_EMIT
  return acc;
}

}  // namespace
}  // namespace cuvs::neighbors::ivf_pq::detail
