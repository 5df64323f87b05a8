/*
 * Pieces shared by the block-per-pair scan kernels (scan_fast.hip, scan_nibble.hip): constant LDS
 * addressing, the LDS-only barrier, and the block's candidate buffer with its pruning step.
 */
#pragma once

#include "device_utils.cuh"
#include "scan_wave_select.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

/* The kernel owns the whole dynamic LDS allocation and has no static LDS, so the allocation starts
 * at LDS address 0.  Addressing it through constants lets the compiler fold every table offset
 * into the immediate field of the ds_read/ds_write instructions.  The first 16 bytes stay unused
 * so that no pointer constant is the (all-ones or zero) null value of the LDS address space. */
#define LDS_AS __attribute__((address_space(3)))
#define GLOBAL_AS __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // one 16-byte chunk of codes
constexpr uint32_t kLdsBase = 16;

constexpr uint32_t kFastCap      = 1536;                // candidate keys held per block (with a 64 KB fp32 table, two blocks still share a CU)
constexpr uint32_t kFastMaxK     = 256;                 // largest k the buffer arithmetic allows
constexpr uint32_t kFastSegIters = (kFastCap - kFastMaxK) / kBlock;  // row iterations per prune

struct fast_tail {
  uint32_t count;
  uint32_t thr;
  uint32_t pad[2];
};

/** Barrier for data exchanged through LDS only: waits for this wave's LDS traffic, not for its
 *  outstanding global loads (the prefetches of the next pair must stay in flight across it). */
__device__ __forceinline__ void lds_barrier()
{
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

/** Keep the k smallest keys of cand[0..count) at the front (in no particular order beyond 64
 *  candidates); publish the k-th score.
 *  `cnt` is the candidate count every thread read between two barriers; returns after a barrier.
 *  No-op when cnt < k. */
__device__ __forceinline__ void block_prune(LDS_AS unsigned long long* cand, LDS_AS fast_tail* tail,
                                            uint32_t k, uint32_t cnt)
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
    lds_barrier();
    return;
  }
  if (cnt <= 1024u) {
    // one wave keeps the k smallest by radix selection on its registers (no order among them)
    if (tid < 64u) {
      const uint32_t kth = cnt <= 256u   ? wave_select_keys<4>(cand, tid, cnt, k)
                           : cnt <= 512u ? wave_select_keys<8>(cand, tid, cnt, k)
                                         : wave_select_keys<16>(cand, tid, cnt, k);
      if (tid == 0) {
        tail->count = k;
        tail->thr   = kth;
      }
    }
    lds_barrier();
    return;
  }
  if (cnt <= 2048u && k <= 256u) {
    // two waves take a half each, then one of them what the halves kept
    const uint32_t second = cnt - 1024u;
    if (tid < 64u) {
      wave_select_keys<16>(cand, tid, 1024u, k);
    } else if (tid < 128u && second > k) {
      wave_select_keys<16>(cand + 1024, tid - 64u, second, k);
    }
    lds_barrier();
    const uint32_t kept = second < k ? second : k;
    unsigned long long moved = kInvalidKey;
    if (tid < kept) { moved = cand[1024u + tid]; }  // kept <= 256 = the block's threads
    lds_barrier();
    if (tid < kept) { cand[k + tid] = moved; }
    lds_barrier();
    if (tid < 64u) {
      const uint32_t kth = wave_select_keys<8>(cand, tid, k + kept, k);
      if (tid == 0) {
        tail->count = k;
        tail->thr   = kth;
      }
    }
    lds_barrier();
    return;
  }
  uint32_t n2 = 128;
  while (n2 < cnt) { n2 <<= 1; }
  for (uint32_t t = cnt + tid; t < n2; t += kBlock) { cand[t] = kInvalidKey; }
  lds_barrier();
  for (uint32_t size = 2; size <= n2; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      for (uint32_t t = tid; t < (n2 >> 1); t += kBlock) {
        const uint32_t pos         = 2 * t - (t & (stride - 1));
        const uint32_t partner     = pos + stride;
        const bool ascending       = (pos & size) == 0;
        const unsigned long long x = cand[pos];
        const unsigned long long y = cand[partner];
        if ((x > y) == ascending) {
          cand[pos]     = y;
          cand[partner] = x;
        }
      }
      lds_barrier();
    }
  }
  if (tid == 0) {
    tail->count = k;
    tail->thr   = uint32_t(cand[k - 1] >> 32);
  }
  lds_barrier();
}

/** 1.0f the optimiser cannot see through: fma(float(h), one, acc) is then selected as a single
 *  v_fma_mix_f32 (convert + add in one instruction) and still equals acc + float(h) exactly. */
__device__ __forceinline__ float opaque_one()
{
  float one = 1.0f;
  asm volatile("" : "+v"(one));
  return one;
}

}  // namespace

}  // namespace cuvs::neighbors::ivf_pq::detail
