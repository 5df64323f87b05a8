/*
 * Persistent LUT + code-scan kernel for 4-bit codes (the sub-byte path of the reference's
 * compute_similarity kernel, cpp/src/neighbors/ivf_pq/detail/jit_lto_kernels/
 * compute_score_impl.cuh:13-79 with PqBits = 4).
 *
 * With 16 entries per subspace a lookup costs the LDS almost nothing (the 64 lanes of a wave hit
 * at most 16 distinct addresses), so the scan is bound by the vector instructions around each
 * lookup.  The kernel keeps them to three per code:
 *
 *   - the table in LDS holds each entry already converted to the accumulator's type (binary16 or
 *     fp32): entry = decode(encode(score)), the value every lookup of the reference decodes again,
 *     so a lookup is followed by one plain add;
 *   - the nibbles of a 32-bit word are turned into byte offsets four at a time
 *     ((w << s) & mask for the even ones, (w >> (4 - s)) & mask for the odd ones), and a code's
 *     table address is one add of a byte of that word to the chunk's table base; the subspace's
 *     offset inside the chunk is an immediate of the LDS read.
 *
 * Organisation as in the 8-bit block kernel: a fixed grid of 256-thread blocks walks the
 * (query, probe) pairs in list order, thread t scores rows t, t + 256, ... of the list, four
 * 16-byte chunks (128 codes) per step with the next step's chunks in flight, the next pair's
 * operands are fetched during the scan of the current one, and candidates go through the block's
 * LDS buffer.  pq_dim is a run-time value (a multiple of 32: whole chunks).
 */
#include "scan_block_select.cuh"

#include <cstdlib>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

constexpr uint32_t kNibStep   = 4;     // 16-byte chunks a thread scores per step
constexpr uint32_t kNibMaxRot = 768;   // rotated dimensions (kNibMaxRot / kBlock staged per thread)
constexpr uint32_t kNibMaxLen = 4;     // dimensions per subspace
constexpr uint32_t kNibRotPer = kNibMaxRot / kBlock;
constexpr uint32_t kNibBookRegs = 48;  // codebook components a thread keeps in registers

/*
 * The lookups of one 32-bit word of codes (8 nibbles), written out instruction by instruction:
 * left to itself the compiler re-derives every nibble from the word with a shift and a mask, adds
 * the table base in two steps and waits for each LDS read before it issues the next.
 *
 *   offs_even / offs_odd   byte offsets (nibble * entry size) of nibbles 0,2,4,6 / 1,3,5,7, one per byte
 *   addr<B>                table base + byte B of such a word, in one SDWA add
 *   read<HALF, IMM>        the LDS read, IMM = the subspace's offset inside the chunk's table
 *   landed<N>              waits until at most N LDS reads are outstanding; the eight registers go
 *                          through it, so the additions that use them cannot be scheduled above it
 */
template <int BYTE>
__device__ __forceinline__ uint32_t nib_addr(uint32_t base, uint32_t offs);
template <>
__device__ __forceinline__ uint32_t nib_addr<0>(uint32_t base, uint32_t offs)
{
  uint32_t a;
  asm volatile("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0"
               : "=v"(a) : "v"(base), "v"(offs));
  return a;
}
template <>
__device__ __forceinline__ uint32_t nib_addr<1>(uint32_t base, uint32_t offs)
{
  uint32_t a;
  asm volatile("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1"
               : "=v"(a) : "v"(base), "v"(offs));
  return a;
}
template <>
__device__ __forceinline__ uint32_t nib_addr<2>(uint32_t base, uint32_t offs)
{
  uint32_t a;
  asm volatile("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2"
               : "=v"(a) : "v"(base), "v"(offs));
  return a;
}
template <>
__device__ __forceinline__ uint32_t nib_addr<3>(uint32_t base, uint32_t offs)
{
  uint32_t a;
  asm volatile("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3"
               : "=v"(a) : "v"(base), "v"(offs));
  return a;
}

template <bool HALF, int IMM>
__device__ __forceinline__ uint32_t nib_read(uint32_t addr)
{
  uint32_t r;
  if (HALF) {
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(IMM));
  } else {
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(IMM));
  }
  return r;
}

template <int N>
__device__ __forceinline__ void nib_landed(uint32_t (&r)[8])
{
  static_assert(N == 0 || N == 8, "one or no word of lookups stays in flight");
  if (N == 8) {
    asm volatile("s_waitcnt lgkmcnt(8)"
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
  } else {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
  }
}

/** Issues the eight lookups of word `w` (word DW of its chunk); `base` = the chunk's table address. */
template <bool HALF, int DW>
__device__ __forceinline__ void nib_issue(uint32_t w, uint32_t base, uint32_t (&r)[8])
{
  constexpr uint32_t SH   = HALF ? 1u : 2u;
  constexpr uint32_t MASK = 0x0F0F0F0Fu << SH;
  constexpr int E         = HALF ? 2 : 4;
  uint32_t even = (w << SH) & MASK;
  uint32_t odd  = (w >> (4u - SH)) & MASK;
  r[0] = nib_read<HALF, (DW * 8 + 0) * 16 * E>(nib_addr<0>(base, even));
  r[1] = nib_read<HALF, (DW * 8 + 1) * 16 * E>(nib_addr<0>(base, odd));
  r[2] = nib_read<HALF, (DW * 8 + 2) * 16 * E>(nib_addr<1>(base, even));
  r[3] = nib_read<HALF, (DW * 8 + 3) * 16 * E>(nib_addr<1>(base, odd));
  r[4] = nib_read<HALF, (DW * 8 + 4) * 16 * E>(nib_addr<2>(base, even));
  r[5] = nib_read<HALF, (DW * 8 + 5) * 16 * E>(nib_addr<2>(base, odd));
  r[6] = nib_read<HALF, (DW * 8 + 6) * 16 * E>(nib_addr<3>(base, even));
  r[7] = nib_read<HALF, (DW * 8 + 7) * 16 * E>(nib_addr<3>(base, odd));
}

/** acc + the eight entries in r, in subspace order. */
template <bool HALF>
__device__ __forceinline__ auto nib_sum(typename std::conditional<HALF, _Float16, float>::type acc,
                                        const uint32_t (&r)[8])
{
  using acc_t = typename std::conditional<HALF, _Float16, float>::type;
#pragma unroll
  for (int i = 0; i < 8; i++) {
    if (HALF) {
      acc = acc_t(acc + acc_t(__builtin_bit_cast(_Float16, uint16_t(r[i]))));
    } else {
      acc = acc_t(acc + acc_t(__uint_as_float(r[i])));
    }
  }
  return acc;
}

/** acc + the 32 entries the codes of one 16-byte chunk select: one word's lookups stay in flight
 *  while the previous word's entries are added. */
template <bool HALF>
__device__ __forceinline__ auto nib_chunk(typename std::conditional<HALF, _Float16, float>::type acc,
                                          const u32x4& codes, uint32_t base)
{
  uint32_t r0[8], r1[8];
  nib_issue<HALF, 0>(codes.x, base, r0);
  nib_issue<HALF, 1>(codes.y, base, r1);
  nib_landed<8>(r0);
  acc = nib_sum<HALF>(acc, r0);
  nib_issue<HALF, 2>(codes.z, base, r0);
  nib_landed<8>(r1);
  acc = nib_sum<HALF>(acc, r1);
  nib_issue<HALF, 3>(codes.w, base, r1);
  nib_landed<8>(r0);
  acc = nib_sum<HALF>(acc, r0);
  nib_landed<0>(r1);
  acc = nib_sum<HALF>(acc, r1);
  return acc;
}

struct nib_prefetch {
  float q[kNibRotPer], c[kNibRotPer];  // rotated query / centre elements tid, tid + 256, ...
  float book[kNibMaxLen];              // per-cluster codebook entry tid % 16
  uint32_t thr;
};

/** decode(encode(score)) in the accumulator's type, for the table type chosen at run time. */
template <bool OUT_HALF, bool IP>
__device__ __forceinline__ auto nib_entry(float score, int lut_dtype)
{
  using acc_t = typename std::conditional<OUT_HALF, _Float16, float>::type;
  if (lut_dtype == CUDA_R_8U) {
    using traits = lut_traits<IP ? LUT_FP8S : LUT_FP8U>;
    const auto e = traits::encode(score);
    if (OUT_HALF) { return acc_t(traits::to_half(e)); }
    return acc_t(traits::to_float(e));
  }
  if (lut_dtype == CUDA_R_16F) {
    using traits = lut_traits<LUT_F16>;
    const auto e = traits::encode(score);
    if (OUT_HALF) { return acc_t(traits::to_half(e)); }
    return acc_t(traits::to_float(e));
  }
  return acc_t(score);  // fp32 table: fp32 accumulator only
}

template <bool OUT_HALF, bool IP, int PQ_LEN>
__global__ __launch_bounds__(kBlock, 2) void scan_nibble_kernel(scan_args a)
{
  using acc_t = typename std::conditional<OUT_HALF, _Float16, float>::type;
  constexpr uint32_t E     = uint32_t(sizeof(acc_t));  // bytes per table entry
  constexpr uint32_t NSUB  = kNibBookRegs / PQ_LEN;    // subspaces a thread can own
  constexpr uint32_t TERMS = IP ? 2u : 1u;             // floats staged per rotated dimension

  const uint32_t rot       = a.rot_dim;
  const uint32_t nch       = a.pq_dim >> 5;  // 16-byte chunks per row
  const uint32_t n16       = a.pq_dim >> 4;  // subspaces a thread owns: t / 16, t / 16 + 16, ...
  const uint32_t n_steps   = (nch + kNibStep - 1u) / kNibStep;
  const uint32_t entries   = a.pq_dim << 4;
  const uint32_t tbl_addr  = kLdsBase;
  const uint32_t diff_addr = tbl_addr + ((entries * E + 15u) & ~15u);
  const uint32_t cand_addr = diff_addr + ((rot * TERMS * 4u + 15u) & ~15u);
  const uint32_t tail_addr = cand_addr + kFastCap * 8u;
  auto* tbl       = reinterpret_cast<LDS_AS acc_t*>(uintptr_t(tbl_addr));
  auto* base_diff = reinterpret_cast<LDS_AS float*>(uintptr_t(diff_addr));
  auto* cand      = reinterpret_cast<LDS_AS unsigned long long*>(uintptr_t(cand_addr));
  auto* tail      = reinterpret_cast<LDS_AS fast_tail*>(uintptr_t(tail_addr));

  const uint32_t tid     = threadIdx.x;
  const uint32_t n_pairs = a.n_pairs_dev != nullptr ? *a.n_pairs_dev : a.n_pairs;
  const uint32_t stride  = gridDim.x;
  if (blockIdx.x >= n_pairs) { return; }  // whole block, before any barrier

  // chunks step * 4 .. step * 4 + 3 of row `row`; past the row's last chunk the last one is read
  // again (never scored), so the loads need no branches
  auto load_step = [&](const uint8_t* list_data, uint32_t row, uint32_t step, u32x4 (&dst)[kNibStep]) {
    const uintptr_t row_base = reinterpret_cast<uintptr_t>(list_data) +
                               uint64_t(row >> 5) * (uint64_t(nch) * 512u) + uint64_t(row & 31u) * 16u;
#pragma unroll
    for (uint32_t m = 0; m < kNibStep; m++) {
      const uint32_t chunk = step * kNibStep + m < nch ? step * kNibStep + m : nch - 1u;
      dst[m] = *reinterpret_cast<const GLOBAL_AS u32x4*>(row_base + uint64_t(chunk) * 512u);
    }
  };
  // the small per-pair operands of pair `d`
  auto fetch_operands = [&](const pair_desc& d, nib_prefetch& f) {
#pragma unroll
    for (uint32_t r = 0; r < kNibRotPer; r++) {
      const uint32_t dim = tid + r * kBlock;
      if (dim < rot) {
        f.q[r] = a.rot_q[uint64_t(d.q) * rot + dim];
        f.c[r] = a.centers_rot[uint64_t(d.label) * rot + dim];
      }
    }
    if (a.per_cluster) {
#pragma unroll
      for (uint32_t t = 0; t < uint32_t(PQ_LEN); t++) {
        f.book[t] = a.pq_centers[(uint64_t(d.label) * PQ_LEN + t) * 16u + (tid & 15u)];
      }
    }
    f.thr = a.query_kth[d.q];
  };
  // first step of the first row of pair `d` (an empty list has no rows to fetch)
  auto fetch = [&](const pair_desc& d, u32x4 (&row0)[kNibStep], nib_prefetch& f) {
    if (d.n_rows != 0) {
      load_step(d.data, tid < d.n_rows ? tid : 0u, 0u, row0);
      fetch_operands(d, f);
    }
  };

  // Thread t builds entry t % 16 of subspaces t / 16, t / 16 + 16, ... of every table, so with
  // per-subspace codebooks the components it needs are the same for every pair: they stay in
  // registers, and a table costs no memory traffic besides the reads of the query / centre terms.
  // (Per-cluster codebooks: the list's entry t % 16 serves every subspace; it comes with the pair.)
  float book[NSUB][PQ_LEN];
  if (!a.per_cluster) {
#pragma unroll
    for (uint32_t i = 0; i < NSUB; i++) {
      if (i < n16) {
#pragma unroll
        for (uint32_t t = 0; t < uint32_t(PQ_LEN); t++) {
          book[i][t] = a.pq_centers[(uint64_t((tid >> 4) + 16u * i) * PQ_LEN + t) * 16u + (tid & 15u)];
        }
      }
    }
  }

  uint32_t it     = blockIdx.x;
  pair_desc cur_d = a.desc[it];
  pair_desc nxt_d = a.desc[it + stride < n_pairs ? it + stride : it];
  u32x4 cur[kNibStep];    // chunks being scored
  u32x4 ahead[kNibStep];  // chunks of the next step, of the next row, or of the next pair's first row
  nib_prefetch cur_f, nxt_f;
#pragma unroll
  for (uint32_t m = 0; m < kNibStep; m++) { cur[m] = u32x4{0u, 0u, 0u, 0u}; ahead[m] = u32x4{0u, 0u, 0u, 0u}; }
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
#pragma unroll
      for (uint32_t r = 0; r < kNibRotPer; r++) {
        const uint32_t dim = tid + r * kBlock;
        if (dim < rot) {
          if (!IP) {
            base_diff[dim] = cur_f.q[r] - cur_f.c[r];
          } else {
            base_diff[2u * dim]      = cur_f.q[r];
            base_diff[2u * dim + 1u] = cur_f.c[r] * cur_f.q[r];
          }
        }
      }
      if (tid == 0) {
        tail->count = 0;
        tail->thr   = 0xFFFFFFFFu;
      }
      if (a.per_cluster) {
#pragma unroll
        for (uint32_t i = 0; i < NSUB; i++) {
#pragma unroll
          for (uint32_t t = 0; t < uint32_t(PQ_LEN); t++) { book[i][t] = cur_f.book[t]; }
        }
      }
      lds_barrier();

      /* ---- lookup table, entries already in the accumulator's type ---- */
      {
        // Groups of 6 subspaces: their query / centre terms are read first, unconditionally
        // (past the thread's last subspace they come from the candidate buffer and are not
        // used), then the arithmetic follows; a read inside the branch that skips the subspaces
        // a thread does not have would expose its latency every time.
        constexpr uint32_t GROUP = 6;
        static_assert(NSUB % GROUP == 0, "whole groups");
        // the thread's first subspace; kept opaque so that the read addresses are formed from it
        // with immediates instead of being precomputed for the whole kernel in registers
        uint32_t own = (tid >> 4) * uint32_t(PQ_LEN) * TERMS;
        asm volatile("" : "+v"(own));
        const LDS_AS float* mine = base_diff + own;
#pragma unroll
        for (uint32_t g = 0; g < NSUB / GROUP; g++) {
          if (g * GROUP < n16) {
            float term[GROUP][PQ_LEN * TERMS];
#pragma unroll
            for (uint32_t u = 0; u < GROUP; u++) {
#pragma unroll
              for (uint32_t x = 0; x < uint32_t(PQ_LEN) * TERMS; x++) {
                term[u][x] = mine[(g * GROUP + u) * 16u * uint32_t(PQ_LEN) * TERMS + x];
              }
            }
#pragma unroll
            for (uint32_t u = 0; u < GROUP; u++) {
              const uint32_t i = g * GROUP + u;
              if (i < n16) {
                float score = 0.0f;
#pragma unroll
                for (uint32_t t = 0; t < uint32_t(PQ_LEN); t++) {
                  const float pqc = book[i][t];
                  if (!IP) {
                    float diff = term[u][t];
                    diff -= pqc;
                    score = fmaf(diff, diff, score);
                  } else {
                    score -= term[u][2u * t + 1u];
                    score = fmaf(-term[u][2u * t], pqc, score);
                  }
                }
                tbl[((tid >> 4) + 16u * i) * 16u + (tid & 15u)] = nib_entry<OUT_HALF, IP>(score, a.lut_dtype);
              }
            }
          }
        }
      }
      lds_barrier();

      /* ---- scan ---- */
      uint32_t thr           = cur_f.thr;
      const uint32_t n_iters = (n_rows + kBlock - 1u) / kBlock;
      for (uint32_t iter = 0; iter < n_iters; iter++) {
        const uint32_t i = iter * kBlock + tid;
        bool valid       = i < n_rows;
        if (valid && list_ids != nullptr) {
          const int64_t id = reinterpret_cast<const GLOBAL_AS int64_t*>(reinterpret_cast<uintptr_t>(list_ids))[i];
          valid = id >= 0 && id < a.filter_nbits && ((a.filter_bits[id >> 5] >> (id & 31)) & 1u) != 0;
        }
        acc_t acc = acc_t(0);
        // whole waves past the end of the list skip the row; L2 sums only grow, so a wave whose
        // rows are all above the bound after a step skips the rest (compute_score's early stop)
        const uint32_t stop_bits = thr >= 0x80000000u ? (thr & 0x7fffffffu) : 0u;
        bool live                = __ballot(valid) != 0ull;
        for (uint32_t step = 0; step < n_steps; step++) {
          // one step in flight: the row's next chunks, the next row's first, or the next pair's.
          // The three cases differ in the address only, so the loads themselves are unconditional
          // (after the last step of the last pair they repeat the current ones).
          const bool more      = step + 1u < n_steps;
          const bool next_row  = !more && iter + 1u < n_iters;
          const bool next_pair = !more && !next_row && has_next && nxt_d.n_rows != 0;
          {
            const uint8_t* src  = next_pair ? nxt_d.data : list_data;
            const uint32_t rows = next_pair ? nxt_d.n_rows : n_rows;
            const uint32_t row  = more ? i : (next_row ? i + kBlock : (next_pair ? tid : i));
            load_step(src, row < rows ? row : 0u, more ? step + 1u : (next_row || next_pair ? 0u : step), ahead);
          }
          if (next_pair) { fetch_operands(nxt_d, nxt_f); }
          if (live) {
#pragma unroll
            for (uint32_t m = 0; m < kNibStep; m++) {
              const uint32_t chunk = step * kNibStep + m;
              if (chunk < nch) {
                // table of the chunk's 32 subspaces (a per-lane copy of a uniform value: the
                // SDWA add takes vector operands)
                uint32_t tb = tbl_addr + chunk * (32u * 16u * E);
                asm volatile("" : "+v"(tb));
                acc = nib_chunk<OUT_HALF>(acc, cur[m], tb);
              }
            }
            if (!IP && more) {
              live = __ballot(valid && !(__float_as_uint(float(acc)) > stop_bits)) != 0ull;
            }
          }
#pragma unroll
          for (uint32_t m = 0; m < kNibStep; m++) { cur[m] = ahead[m]; }
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
        if (iter + 1u < n_iters && (iter + 1u) % kFastSegIters == 0u) {
          lds_barrier();
          const uint32_t seg_cnt = tail->count;
          lds_barrier();
          block_prune(cand, tail, a.k, seg_cnt);
          const uint32_t t2 = tail->thr;
          thr               = t2 < thr ? t2 : thr;
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
    if (n_rows == 0) {
#pragma unroll
      for (uint32_t m = 0; m < kNibStep; m++) { cur[m] = ahead[m]; }
    }
    it += stride;
    cur_d = nxt_d;
    nxt_d = after_d;
    cur_f = nxt_f;
  }
}

size_t nibble_smem(const scan_args& a, bool out_half)
{
  const bool ip    = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  const size_t tbl = (size_t(a.pq_dim) * 16 * (out_half ? 2 : 4) + 15) & ~size_t(15);
  const size_t dif = (size_t(a.rot_dim) * (ip ? 2 : 1) * 4 + 15) & ~size_t(15);
  return kLdsBase + tbl + dif + size_t(kFastCap) * 8 + sizeof(fast_tail);
}

template <bool OUT_HALF, bool IP, int PQ_LEN>
void launch_nibble_instance(const scan_args& a, hipStream_t stream)
{
  auto kernel       = scan_nibble_kernel<OUT_HALF, IP, PQ_LEN>;
  const size_t smem = nibble_smem(a, OUT_HALF);
  // per instance: the LDS limit once; the occupancy depends on the table size (pq_dim) and is asked
  // at every launch (a host-side computation)
  static const int attr_set = [&] {
    CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
    return 1;
  }();
  (void)attr_set;
  int occ = 0;
  CUVS_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, kBlock, smem));
  const uint32_t known_grid = uint32_t(occ > 0 ? occ : 1) * uint32_t(device_cu_count());
  uint32_t grid = known_grid;
  if (a.n_pairs_dev == nullptr) {
    if (grid > a.n_pairs) { grid = a.n_pairs; }
    if (grid == 0) { return; }
  }
  kernel<<<grid, kBlock, smem, stream>>>(a);
  CUVS_HIP_TRY(hipGetLastError());
}

template <bool OUT_HALF, bool IP>
void launch_nibble_len(const scan_args& a, hipStream_t stream)
{
  if (a.pq_len == 1) { launch_nibble_instance<OUT_HALF, IP, 1>(a, stream); }
  if (a.pq_len == 2) { launch_nibble_instance<OUT_HALF, IP, 2>(a, stream); }
  if (a.pq_len == 4) { launch_nibble_instance<OUT_HALF, IP, 4>(a, stream); }
}

}  // namespace

bool scan_nibble_supported(const scan_args& a)
{
  if (!a.fused || a.pq_bits != 4 || a.k > kFastMaxK) { return false; }
  if (a.pq_dim % 32u != 0 || a.rot_dim != a.pq_dim * a.pq_len) { return false; }
  if (a.pq_len != 1 && a.pq_len != 2 && a.pq_len != 4) { return false; }
  // the codebook components a thread owns fit its registers
  if ((a.pq_dim >> 4) * a.pq_len > kNibBookRegs || a.rot_dim > kNibMaxRot) { return false; }
  if (a.lut_dtype == CUDA_R_32F && a.out_half) { return false; }
  return nibble_smem(a, a.out_half) <= 64 * 1024;
}

bool launch_scan_nibble(const scan_args& a, hipStream_t stream)
{
  if (!scan_nibble_supported(a) || a.n_queries == 0 || a.desc == nullptr) { return false; }
  const bool ip = a.metric == int(DistanceType::InnerProduct) || a.metric == int(DistanceType::CosineExpanded);
  if (a.out_half) {
    if (ip) { launch_nibble_len<true, true>(a, stream); } else { launch_nibble_len<true, false>(a, stream); }
  } else {
    if (ip) { launch_nibble_len<false, true>(a, stream); } else { launch_nibble_len<false, false>(a, stream); }
  }
  return true;
}

}  // namespace cuvs::neighbors::ivf_pq::detail
