/*
 * Device-side helpers shared by the HIP translation units: ordered float keys, wave scans,
 * block-wide bitonic sort, exact k-smallest selection, lookup-table element types.
 */
#pragma once

#include "detail.hpp"

#include <hip/hip_runtime.h>

#include <cfloat>
#include <type_traits>

namespace cuvs::neighbors::ivf_pq::detail {
namespace {

constexpr int kBlock              = 256;
constexpr unsigned long long kInvalidKey = 0xFFFFFFFFFFFFFFFFull;

/* ---------------------------------------------------------------------------------------- */
/* small device helpers                                                                      */
/* ---------------------------------------------------------------------------------------- */

/** Compute units of the current device, asked once per process (function-local statics are
 *  initialised exactly once also when several host threads make their first call together). */
inline int device_cu_count()
{
  static const int n = [] {
    int dev = 0, count = 0;
    CUVS_HIP_TRY(hipGetDevice(&dev));
    CUVS_HIP_TRY(hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, dev));
    return count;
  }();
  return n;
}

/** Raises the kernel's dynamic LDS limit to `smem_limit` and returns how many blocks of `block`
 *  threads with `smem` bytes of dynamic LDS fit one compute unit (at least 1).  Meant to initialise
 *  a `static const int` of the launcher of one kernel instance. */
template <typename Kernel>
inline int prepare_persistent_kernel(Kernel kernel, int block, size_t smem, size_t smem_limit)
{
  CUVS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, int(smem_limit)));
  int occ = 0;
  CUVS_HIP_TRY(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, kernel, block, smem));
  return occ > 0 ? occ : 1;
}

/** Monotone map float -> uint32 (ascending); -0 and +0 map to the same key. */
__device__ __forceinline__ uint32_t order_f32(float f)
{
  f          = (f == 0.0f) ? 0.0f : f;
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float unorder_f32(uint32_t k)
{
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

__device__ __forceinline__ uint32_t next_pow2_dev(uint32_t v)
{
  return v <= 1u ? 1u : 1u << (32 - __builtin_clz(v - 1u));
}

__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v)
{
  const uint32_t lane = threadIdx.x & 63u;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    uint32_t o = __shfl_up(v, d, 64);
    if (lane >= uint32_t(d)) { v += o; }
  }
  return v;
}

/** In-place ascending bitonic sort of n (power of two) keys in LDS by the whole block. */
template <typename KeyPtr>
__device__ void block_bitonic_sort(KeyPtr a, uint32_t n)
{
  for (uint32_t size = 2; size <= n; size <<= 1) {
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      for (uint32_t t = threadIdx.x; t < (n >> 1); t += blockDim.x) {
        const uint32_t pos     = 2 * t - (t & (stride - 1));
        const uint32_t partner = pos + stride;
        const bool ascending   = (pos & size) == 0;
        const unsigned long long x = a[pos];
        const unsigned long long y = a[partner];
        if ((x > y) == ascending) {
          a[pos]     = y;
          a[partner] = x;
        }
      }
      __syncthreads();
    }
  }
}

/* ---------------------------------------------------------------------------------------- */
/* exact k-smallest selection of 64-bit keys by one block: MSB-first radix passes over an     */
/* 11-bit digit that stop as soon as a digit boundary coincides with the k-th element, then    */
/* one collection pass and a bitonic sort of the k survivors.                                  */
/* ---------------------------------------------------------------------------------------- */

constexpr int kRadixBits = 11;
constexpr int kBins      = 1 << kRadixBits;

struct select_smem {
  uint32_t hist[kBins];
  uint32_t wave_sums[kBlock / 64];
  uint32_t bin, before, upto, count;
};

/**
 * key_of(i), i < n, returns the key of element i or kInvalidKey.  Writes the min(k, #valid)
 * smallest keys ascending into out[0..), pads the rest of out[0..out_cap) with kInvalidKey and
 * returns their number.  out_cap is a power of two >= k.  All threads of the block must call.
 */
template <typename KeyFn>
__device__ uint32_t block_select_sorted(KeyFn key_of, uint32_t n, uint32_t k,
                                        unsigned long long* out, uint32_t out_cap, select_smem& sm)
{
  const uint32_t tid = threadIdx.x;
  unsigned long long prefix = 0;
  uint32_t pb   = 0;  // number of leading key bits already fixed in `prefix`
  uint32_t need = k;
  bool none     = false;
  for (;;) {
    const uint32_t digit_bits = (64u - pb) < uint32_t(kRadixBits) ? (64u - pb) : uint32_t(kRadixBits);
    const uint32_t shift      = 64u - pb - digit_bits;
    const uint32_t dmask      = (1u << digit_bits) - 1u;
    for (uint32_t i = tid; i < uint32_t(kBins); i += kBlock) { sm.hist[i] = 0; }
    __syncthreads();
    for (uint32_t i = tid; i < n; i += kBlock) {
      const unsigned long long key = key_of(i);
      if (key != kInvalidKey && (pb == 0 || (key >> (64u - pb)) == prefix)) {
        atomicAdd(&sm.hist[uint32_t(key >> shift) & dmask], 1u);
      }
    }
    __syncthreads();
    constexpr uint32_t per = kBins / kBlock;
    uint32_t s = 0;
#pragma unroll
    for (uint32_t j = 0; j < per; j++) { s += sm.hist[tid * per + j]; }
    uint32_t incl = wave_inclusive_scan(s);
    if ((tid & 63u) == 63u) { sm.wave_sums[tid >> 6] = incl; }
    __syncthreads();
    uint32_t base = 0, total = 0;
#pragma unroll
    for (uint32_t w = 0; w < kBlock / 64; w++) {
      const uint32_t ws = sm.wave_sums[w];
      if (w < (tid >> 6)) { base += ws; }
      total += ws;
    }
    incl += base;
    const uint32_t excl = incl - s;
    if (pb == 0 && need > total) { need = total; }
    if (need == 0) {
      none = true;
      break;
    }
    if (excl < need && need <= incl) {
      uint32_t c = excl;
      for (uint32_t j = 0; j < per; j++) {
        const uint32_t h = sm.hist[tid * per + j];
        if (c + h >= need) {
          sm.bin    = tid * per + j;
          sm.before = c;
          sm.upto   = c + h;
          break;
        }
        c += h;
      }
    }
    __syncthreads();
    const uint32_t b      = sm.bin;
    const uint32_t before = sm.before;
    const uint32_t upto   = sm.upto;
    prefix                = (prefix << digit_bits) | b;
    pb += digit_bits;
    __syncthreads();
    if (upto == need || pb >= 64u) { break; }
    need -= before;
  }

  if (tid == 0) { sm.count = 0; }
  __syncthreads();
  if (!none) {
    for (uint32_t i = tid; i < n; i += kBlock) {
      const unsigned long long key = key_of(i);
      if (key != kInvalidKey && (key >> (64u - pb)) <= prefix) {
        const uint32_t pos = atomicAdd(&sm.count, 1u);
        if (pos < out_cap) { out[pos] = key; }
      }
    }
  }
  __syncthreads();
  uint32_t cnt = sm.count;
  if (cnt > out_cap) { cnt = out_cap; }
  for (uint32_t i = cnt + tid; i < out_cap; i += kBlock) { out[i] = kInvalidKey; }
  __syncthreads();
  block_bitonic_sort(out, out_cap);
  return cnt < k ? cnt : k;
}

/**
 * The same result for k <= kBlock, in one or two passes over the keys: thread t takes keys t,
 * t + kBlock, ... (up to kMinimaPer of them stay in registers; more are read a second time); the
 * k-th smallest of the kBlock per-thread minima (by the keys' high words) is at or above the k-th
 * smallest key, and for keys in no particular order only a few more than k lie at or below it;
 * those are collected in LDS (the histogram area of `sm`) and ranked.  Returns false, with nothing
 * written, when more than 1024 keys pass the bound (keys in an adversarial order, or k close to the
 * number of threads' worth of valid keys): the caller then selects by radix passes.
 */
constexpr uint32_t kMinimaPer = 16;
template <typename KeyFn>
__device__ bool block_select_by_minima(KeyFn key_of, uint32_t n, uint32_t k, unsigned long long* out,
                                       uint32_t out_cap, select_smem& sm)
{
  static_assert(sizeof(sm.hist) >= 1024 * sizeof(unsigned long long), "candidate area");
  constexpr uint32_t kCap = 1024;
  __shared__ uint32_t mins[kBlock];
  __shared__ uint32_t s_bound, s_count;
  unsigned long long* cand = reinterpret_cast<unsigned long long*>(sm.hist);
  const uint32_t tid  = threadIdx.x;
  const uint32_t lane = tid & 63u;
  const uint32_t wid  = tid >> 6;
  const bool held = n <= kBlock * kMinimaPer;  // uniform
  unsigned long long key[kMinimaPer];
  uint32_t mine = 0xFFFFFFFFu;
  if (held) {
#pragma unroll
    for (uint32_t j = 0; j < kMinimaPer; j++) {
      const uint32_t i = j * kBlock + tid;
      key[j]           = i < n ? key_of(i) : kInvalidKey;
    }
#pragma unroll
    for (uint32_t j = 0; j < kMinimaPer; j++) {
      const uint32_t hi = uint32_t(key[j] >> 32);
      mine              = hi < mine ? hi : mine;
    }
  } else {
    // one block may be the only one with this many keys, so what bounds it is the number of
    // requests it keeps in flight: sixteen per thread here, eight where whole keys come back
    constexpr uint32_t kAhead = 16;
    for (uint32_t i0 = tid; i0 < n; i0 += kAhead * kBlock) {
      uint32_t hi[kAhead];
#pragma unroll
      for (uint32_t u = 0; u < kAhead; u++) {
        const uint32_t i = i0 + u * kBlock;
        hi[u]            = i < n ? uint32_t(key_of(i) >> 32) : 0xFFFFFFFFu;
      }
#pragma unroll
      for (uint32_t u = 0; u < kAhead; u++) { mine = hi[u] < mine ? hi[u] : mine; }
    }
  }
  if (tid == 0) {
    s_bound = 0xFFFFFFFFu;
    s_count = 0;
  }
  // ascending bitonic sort of the wave's 64 minima
  uint32_t v = mine;
#pragma unroll
  for (uint32_t size = 2; size <= 64; size <<= 1) {
#pragma unroll
    for (uint32_t stride = size >> 1; stride > 0; stride >>= 1) {
      const uint32_t other = __shfl_xor(v, int(stride), 64);
      const bool ascending = (lane & size) == 0 || size == 64;
      const bool low_half  = (lane & stride) == 0;
      const uint32_t lo    = v < other ? v : other;
      const uint32_t hi    = v < other ? other : v;
      v                    = (low_half == ascending) ? lo : hi;
    }
  }
  mins[tid] = v;
  __syncthreads();
  // rank of (v, wid, lane) among all minima: `<=` against earlier waves' lists
  uint32_t rank = lane;
#pragma unroll
  for (uint32_t w = 0; w < kBlock / 64; w++) {
    if (w == wid) { continue; }
    const uint32_t* list = mins + w * 64u;
    uint32_t lo = 0, hi = 64;
#pragma unroll
    for (int step = 0; step < 6; step++) {
      const uint32_t mid = (lo + hi) >> 1;
      const uint32_t m   = list[mid];
      const bool before  = w < wid ? m <= v : m < v;
      lo                 = before ? mid + 1u : lo;
      hi                 = before ? hi : mid;
    }
    rank += lo;
  }
  if (rank == k - 1u) { s_bound = v; }
  __syncthreads();
  const uint32_t bound = s_bound;
  if (mine <= bound) {
    if (held) {
#pragma unroll
      for (uint32_t j = 0; j < kMinimaPer; j++) {
        if (key[j] != kInvalidKey && uint32_t(key[j] >> 32) <= bound) {
          const uint32_t pos = atomicAdd(&s_count, 1u);
          if (pos < kCap) { cand[pos] = key[j]; }
        }
      }
    } else {
      constexpr uint32_t kAhead = 8;
      for (uint32_t i0 = tid; i0 < n; i0 += kAhead * kBlock) {
        unsigned long long again[kAhead];
#pragma unroll
        for (uint32_t u = 0; u < kAhead; u++) {
          const uint32_t i = i0 + u * kBlock;
          again[u]         = i < n ? key_of(i) : kInvalidKey;
        }
#pragma unroll
        for (uint32_t u = 0; u < kAhead; u++) {
          if (again[u] != kInvalidKey && uint32_t(again[u] >> 32) <= bound) {
            const uint32_t pos = atomicAdd(&s_count, 1u);
            if (pos < kCap) { cand[pos] = again[u]; }
          }
        }
      }
    }
  }
  __syncthreads();
  const uint32_t total = s_count;
  __syncthreads();  // everybody has read the count before a later call resets it
  if (total > kCap) { return false; }
  if (total <= kBlock) {
    // few candidates: place each by counting the smaller ones (keys are distinct)
    unsigned long long mykey = kInvalidKey;
    uint32_t pos             = 0;
    if (tid < total) {
      mykey = cand[tid];
      for (uint32_t x = 0; x < total; x++) { pos += cand[x] < mykey ? 1u : 0u; }
    }
    for (uint32_t r = tid; r < out_cap; r += kBlock) { out[r] = kInvalidKey; }
    __syncthreads();
    if (tid < total && pos < out_cap) { out[pos] = mykey; }
    __syncthreads();
  } else {
    uint32_t n_sort = 1;
    while (n_sort < total) { n_sort <<= 1; }
    for (uint32_t i = total + tid; i < n_sort; i += kBlock) { cand[i] = kInvalidKey; }
    __syncthreads();
    block_bitonic_sort(cand, n_sort);
    for (uint32_t r = tid; r < out_cap; r += kBlock) { out[r] = r < total ? cand[r] : kInvalidKey; }
    __syncthreads();
  }
  return true;
}

/* ---------------------------------------------------------------------------------------- */
/* lookup-table element types                                                                */
/* ---------------------------------------------------------------------------------------- */

enum { LUT_F32 = 0, LUT_F16 = 1, LUT_FP8U = 2, LUT_FP8S = 3 };

/* 8-bit float with 5 exponent bits, bias 15, 3 (unsigned) or 2 (signed, sign in the LSB) value
 * bits: encode truncates, decode adds half a unit (cuVS ivf_pq_fp_8bit.cuh:31-100). */
__device__ __forceinline__ uint8_t fp8_encode_unsigned(float v)
{
  // Reference form: v < 2^-15 -> 0; v >= 2^16 * (2 - 1/8) -> 0xff; else
  // (bits(v) + (15 << 23) - 0x3f800000) >> 20.  With the bit pattern read as a signed integer
  // (negative floats are negative integers, positive floats order like their patterns) this is
  // clamp(bits(v) - bits(2^-15), 0, 0x0fffffff) >> 20, which needs no branches.
  const int x = int(__float_as_uint(v)) - 0x38000000;
  const int c = x < 0 ? 0 : (x > 0x0fffffff ? 0x0fffffff : x);
  return uint8_t(uint32_t(c) >> 20);
}
__device__ __forceinline__ uint8_t fp8_encode_signed(float v)
{
  const uint8_t u = fp8_encode_unsigned(fabsf(v));
  return uint8_t((u & 0xfeu) | (v < 0.0f ? 1u : 0u));
}

template <int LUT>
struct lut_traits;
template <>
struct lut_traits<LUT_F32> {
  using storage = float;
  static __device__ __forceinline__ storage encode(float v) { return v; }
  static __device__ __forceinline__ float to_float(storage s) { return s; }
  static __device__ __forceinline__ _Float16 to_half(storage s) { return _Float16(s); }
};
template <>
struct lut_traits<LUT_F16> {
  using storage = _Float16;
  static __device__ __forceinline__ storage encode(float v)
  {
    // The table entry is the fp32 score rounded to binary16.  Without this barrier the compiler
    // folds the last FMA of the score and the conversion into v_fma_mixlo_f16, which rounds the
    // exact FMA result straight to binary16 (one rounding instead of two) and changes values.
    asm volatile("" : "+v"(v));
    return _Float16(v);
  }
  static __device__ __forceinline__ float to_float(storage s) { return float(s); }
  static __device__ __forceinline__ _Float16 to_half(storage s) { return s; }
};
template <>
struct lut_traits<LUT_FP8U> {
  using storage = uint8_t;
  static __device__ __forceinline__ storage encode(float v) { return fp8_encode_unsigned(v); }
  static __device__ __forceinline__ float to_float(storage s)
  {
    return __uint_as_float(0x38080000u + (uint32_t(s) << 20));
  }
  static __device__ __forceinline__ _Float16 to_half(storage s)
  {
    const uint16_t bits = uint16_t(0x0040u + (uint32_t(s) << 7));
    return __builtin_bit_cast(_Float16, bits);
  }
};
template <>
struct lut_traits<LUT_FP8S> {
  using storage = uint8_t;
  static __device__ __forceinline__ storage encode(float v) { return fp8_encode_signed(v); }
  static __device__ __forceinline__ float to_float(storage s)
  {
    const uint32_t bits = 0x38080000u + (uint32_t(s & 0xfeu) << 20);
    return __uint_as_float(bits | (uint32_t(s & 1u) << 31));
  }
  static __device__ __forceinline__ _Float16 to_half(storage s)
  {
    const uint16_t bits = uint16_t((0x0040u + (uint32_t(s & 0xfeu) << 7)) | (uint32_t(s & 1u) << 15));
    return __builtin_bit_cast(_Float16, bits);
  }
};

__device__ __forceinline__ bool is_ip_metric(int metric)
{
  return metric == int(DistanceType::InnerProduct) || metric == int(DistanceType::CosineExpanded);
}


}  // namespace
}  // namespace cuvs::neighbors::ivf_pq::detail
