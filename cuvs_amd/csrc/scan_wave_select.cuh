/*
 * Selection of the k smallest of a wave's candidate keys in registers: ballots and counts only, no
 * LDS round trips.  For the scan kernels that keep one candidate buffer per wave.
 */
#pragma once

#include "device_utils.cuh"

#include <type_traits>

namespace cuvs::neighbors::ivf_pq::detail {

namespace {

#ifndef LDS_AS
#define LDS_AS __attribute__((address_space(3)))
#define GLOBAL_AS __attribute__((address_space(1)))
#endif

/** Largest value of the wave (unsigned; lanes that take no part pass 0): prefix maxima inside the
 *  rows of 16 lanes, then across the rows; lane 63 ends up with the result. */
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
  auto step = [&](auto ctrl, auto rows) {
    const uint32_t other = uint32_t(__builtin_amdgcn_update_dpp(0, int(v), decltype(ctrl)::value, decltype(rows)::value, 0xf, false));
    v                    = other > v ? other : v;
  };
  step(std::integral_constant<int, 0x111>{}, std::integral_constant<int, 0xf>{});  // row_shr:1
  step(std::integral_constant<int, 0x112>{}, std::integral_constant<int, 0xf>{});  // row_shr:2
  step(std::integral_constant<int, 0x114>{}, std::integral_constant<int, 0xf>{});  // row_shr:4
  step(std::integral_constant<int, 0x118>{}, std::integral_constant<int, 0xf>{});  // row_shr:8
  step(std::integral_constant<int, 0x142>{}, std::integral_constant<int, 0xa>{});  // row_bcast:15 into rows 1, 3
  step(std::integral_constant<int, 0x143>{}, std::integral_constant<int, 0xc>{});  // row_bcast:31 into rows 2, 3
  return uint32_t(__builtin_amdgcn_readlane(int(v), 63));
}

/** Binary radix selection of the r smallest (r >= 1) of the wave's values value[j] of the lanes in
 *  live[j], which are at least r, from bit `top` down (all the values agree above it and `prefix`
 *  holds those bits).  Ballots and counts only: the state is scalar and nothing goes through LDS.
 *  Ends as soon as a group of exactly the right size is split off: then the r smallest are the
 *  values v with (v >> bit) <= (prefix >> bit) for the returned bit.  Otherwise returns -1 and
 *  prefix is the r-th smallest value itself (which may occur several times). */
template <int NK>
__device__ __forceinline__ int wave_radix_select(const uint32_t (&value)[NK], const unsigned long long (&live)[NK],
                                                 uint32_t r, int top, uint32_t& prefix)
{
#pragma unroll 1
  for (int bit = top; bit >= 0; bit--) {
    // values that share the decided bits and have a zero at `bit`
    uint32_t zeros = 0;
#pragma unroll
    for (int j = 0; j < NK; j++) {
      zeros += uint32_t(__popcll(__builtin_amdgcn_ballot_w64((value[j] >> bit) == (prefix >> bit)) & live[j]));
    }
    if (zeros == r) { return bit; }
    if (zeros < r) {
      r -= zeros;
      prefix |= 1u << bit;
    }
  }
  return -1;
}

/** The r-th smallest (r >= 1) of the wave's values value[j] of the lanes in live[j] (at least r of
 *  them; lane 0 of value[0] must be one).  The bits that all values share are skipped, and the
 *  selection ends as soon as a group of exactly the right size is split off, whose largest member
 *  is the answer. */
template <int NK>
__device__ __forceinline__ uint32_t wave_kth_smallest(const uint32_t (&value)[NK], const unsigned long long (&live)[NK],
                                                      uint32_t r, uint32_t lane)
{
  const uint32_t first = uint32_t(__builtin_amdgcn_readfirstlane(int(value[0])));
  uint32_t differ      = 0;
#pragma unroll
  for (int j = 0; j < NK; j++) { differ |= ((live[j] >> lane) & 1ull) != 0ull ? value[j] ^ first : 0u; }
  int top = -1;  // highest bit set in any lane's `differ`
  if (__builtin_amdgcn_ballot_w64(differ != 0u) != 0ull) {
    top = 0;
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1) {
      if (__builtin_amdgcn_ballot_w64((differ >> (top + s)) != 0u) != 0ull) { top += s; }
    }
  }
  uint32_t kth  = top >= 0 ? (first >> top >> 1 << top << 1) : first;  // the common bits
  const int cut = wave_radix_select<NK>(value, live, r, top, kth);
  if (cut < 0) { return kth; }
  uint32_t largest = 0;
#pragma unroll
  for (int j = 0; j < NK; j++) {
    const bool in = ((live[j] >> lane) & 1ull) != 0ull && (value[j] >> cut) <= (kth >> cut);
    largest       = in && value[j] > largest ? value[j] : largest;
  }
  return wave_max_u32(largest);
}

/** Keeps the k smallest of the first n >= k keys (n <= 64 * NK) of one wave's buffer, in buf[0 .. k)
 *  in no particular order, and returns the high word of the k-th smallest.  Keys are distinct (the
 *  low word numbers the sample); among equal high words the smaller low words win, as in a sort of
 *  the whole keys.  The keys sit in registers while the selection runs; LDS operations of a wave
 *  execute in program order, so the compacting writes come after every read. */
template <int NK>
__device__ __forceinline__ uint32_t wave_select_keys(LDS_AS unsigned long long* buf, uint32_t lane, uint32_t n, uint32_t k)
{
  unsigned long long key[NK], live[NK];
  uint32_t hi[NK], lo[NK];
#pragma unroll
  for (int j = 0; j < NK; j++) {
    const bool in = uint32_t(j) * 64u + lane < n;
    live[j]       = __builtin_amdgcn_ballot_w64(in);
    key[j]        = in ? buf[uint32_t(j) * 64u + lane] : 0ull;
    hi[j]         = uint32_t(key[j] >> 32);
    lo[j]         = uint32_t(key[j]);
  }
  // the bits in which the high words differ at all: scores of one pair share their leading bits
  const uint32_t first = uint32_t(__builtin_amdgcn_readfirstlane(int(hi[0])));  // lane 0 holds a key: n >= 1
  uint32_t differ      = 0;
#pragma unroll
  for (int j = 0; j < NK; j++) { differ |= uint32_t(j) * 64u + lane < n ? hi[j] ^ first : 0u; }
  int top = -1;  // highest bit set in any lane's `differ`
  if (__builtin_amdgcn_ballot_w64(differ != 0u) != 0ull) {
    top = 0;
#pragma unroll
    for (int s = 16; s >= 1; s >>= 1) {
      if (__builtin_amdgcn_ballot_w64((differ >> (top + s)) != 0u) != 0ull) { top += s; }
    }
  }
  uint32_t kth  = top >= 0 ? (first >> top >> 1 << top << 1) : first;  // the common bits
  const int cut = wave_radix_select<NK>(hi, live, k, top, kth);
  bool keep[NK];
  if (cut >= 0) {
    // exactly k keys lie at or below the group that was split off; its largest is the k-th
    uint32_t largest = 0;
#pragma unroll
    for (int j = 0; j < NK; j++) {
      keep[j] = uint32_t(j) * 64u + lane < n && (hi[j] >> cut) <= (kth >> cut);
      largest = keep[j] && hi[j] > largest ? hi[j] : largest;
    }
    kth = wave_max_u32(largest);
  } else {
    uint32_t less = 0, ties = 0;
    unsigned long long tied[NK];
#pragma unroll
    for (int j = 0; j < NK; j++) {
      tied[j] = __builtin_amdgcn_ballot_w64(hi[j] == kth) & live[j];
      less += uint32_t(__popcll(__builtin_amdgcn_ballot_w64(hi[j] < kth) & live[j]));
      ties += uint32_t(__popcll(tied[j]));
    }
    // of the keys whose high word is kth, those with low words up to here are kept
    uint32_t last_low = 0xFFFFFFFFu;
    if (less + ties > k) {
      last_low      = 0;
      const int at  = wave_radix_select<NK>(lo, tied, k - less, 31, last_low);
      if (at >= 0) { last_low |= (1u << at) - 1u; }  // every low word of the group that was split off
    }
#pragma unroll
    for (int j = 0; j < NK; j++) {
      keep[j] = uint32_t(j) * 64u + lane < n && (hi[j] < kth || (hi[j] == kth && lo[j] <= last_low));
    }
  }
  uint32_t base = 0;
#pragma unroll
  for (int j = 0; j < NK; j++) {
    const unsigned long long mask = __builtin_amdgcn_ballot_w64(keep[j]);
    const uint32_t below = __builtin_amdgcn_mbcnt_hi(uint32_t(mask >> 32), __builtin_amdgcn_mbcnt_lo(uint32_t(mask), 0u));
    if (keep[j]) { buf[base + below] = key[j]; }
    base += uint32_t(__popcll(mask));
  }
  return kth;
}

}  // namespace
}  // namespace cuvs::neighbors::ivf_pq::detail
