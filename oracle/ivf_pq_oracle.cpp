/*
 * CPU oracle for IVF-PQ search -- TEST INFRASTRUCTURE ONLY (see ivf_pq_oracle.h).
 *
 * Restates, in plain scalar C++, what cuVS computes on the path
 *   cuvs::neighbors::ivf_pq::search  (cpp/src/neighbors/ivf_pq/ivf_pq_search.cuh:878-1048).
 * Each function cites the reference lines it follows.  Where the reference leaves
 * the arithmetic to a library whose source is not part of the reference tree
 * (cuBLAS GEMM summation order, RAFT select_k tie-breaking, nvcc's FMA contraction)
 * this file fixes one deterministic choice and says so:
 *
 *   - dot products accumulate in fp32 with fused multiply-add, ascending index
 *     (parity unpinned: the reference's GEMM order is unspecified);
 *   - `score += d*d` in the lookup-table construction is one fused multiply-add
 *     (parity unpinned: nvcc's default contraction);
 *   - every top-k keeps the k smallest by (score, index) and reports them ascending
 *     (parity unpinned: the reference documents the row order as unspecified).
 *
 * Pinned parts (checked in tests/ against closed forms, numpy and brute force):
 * the fp_8bit codec, IEEE half conversion/addition, the interleaved list layout,
 * the lookup-table + scan identity  sum_j LUT[j][code_j] == ||(q - c) - decode(codes)||^2,
 * coarse selection vs. textbook L2, chunk indices vs. cumsum, id translation vs. searchsorted,
 * distance post-processing; the reduced-precision coarse scores: coarse_scores_f16 against numpy's
 * float16 roundings around an fp32 FMA chain (and an exact-integer case), coarse_scores_i8 against
 * the published formulas restated in numpy (tests/test_oracle_search.py).
 */
#include "ivf_pq_oracle.h"

#include <algorithm>
#include <atomic>
#include <cfloat>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <limits>
#include <string>
#include <thread>
#include <utility>
#include <vector>

namespace {

thread_local std::string g_error;

inline uint32_t f2u(float f)
{
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
inline float u2f(uint32_t u)
{
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}

/* ---------------- IEEE binary16, round-to-nearest-even ---------------- */

uint16_t float_to_half(float f)
{
  const uint32_t x    = f2u(f);
  const uint16_t sign = uint16_t((x >> 16) & 0x8000u);
  const uint32_t a    = x & 0x7fffffffu;
  if (a > 0x7f800000u) { return uint16_t(sign | 0x7e00u | ((a >> 13) & 0x3ffu)); }  // NaN
  if (a >= 0x47800000u) { return uint16_t(sign | 0x7c00u); }  // >= 65536 (and inf) -> inf
  if (a < 0x38800000u) {
    // below the smallest normal half (2^-14): result is a multiple of 2^-24
    const uint32_t e = a >> 23;
    if (e < 102u) { return sign; }  // < 2^-25 rounds to zero
    const uint32_t mant  = (a & 0x7fffffu) | 0x800000u;
    const uint32_t shift = 126u - e;  // 14..24
    uint32_t r           = mant >> shift;
    const uint32_t rem   = mant & ((1u << shift) - 1u);
    const uint32_t halfw = 1u << (shift - 1u);
    if (rem > halfw || (rem == halfw && (r & 1u))) { r++; }
    return uint16_t(sign | r);
  }
  uint32_t r         = (((a >> 23) - 112u) << 10) | ((a & 0x7fffffu) >> 13);
  const uint32_t rem = a & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) { r++; }  // may carry up to inf
  return uint16_t(sign | r);
}

float half_to_float(uint16_t h)
{
  const uint32_t sign = uint32_t(h & 0x8000u) << 16;
  const uint32_t e    = (h >> 10) & 0x1fu;
  const uint32_t m    = h & 0x3ffu;
  if (e == 0x1fu) { return u2f(sign | 0x7f800000u | (m << 13)); }
  if (e == 0) {
    const float v = float(m) * 5.9604644775390625e-08f;  // m * 2^-24, exact
    return (sign != 0) ? -v : v;
  }
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* a + b in binary16.  fp32 carries 24 >= 2*11+2 significand bits, so rounding the fp32 sum to
 * half equals the correctly rounded half sum. */
inline uint16_t half_add(uint16_t a, uint16_t b)
{
  return float_to_half(half_to_float(a) + half_to_float(b));
}

/* ---------------- fp_8bit<5, Signed>  (ivf_pq_fp_8bit.cuh:31-100) ---------------- */

constexpr uint32_t kFp8ExpBits = 5;
constexpr uint32_t kFp8ExpMask = (1u << (kFp8ExpBits - 1u)) - 1u;  // 15
constexpr uint32_t kFp8ValBits = 8u - kFp8ExpBits;                 // 3

uint8_t fp8_encode_unsigned(float v)
{
  const float kMin = 1.0f / float(1u << kFp8ExpMask);
  const float kMax = float(1u << (kFp8ExpMask + 1)) * (2.0f - 1.0f / float(1u << kFp8ValBits));
  if (v < kMin) { return 0; }  // small and negative values collapse to zero
  if (v >= kMax) { return 0xffu; }
  return uint8_t((f2u(v) + (kFp8ExpMask << 23u) - 0x3f800000u) >> (15u + kFp8ExpBits));
}

uint8_t fp8_encode(float v, bool is_signed)
{
  if (!is_signed) { return fp8_encode_unsigned(v); }
  uint8_t u = fp8_encode_unsigned(std::fabs(v));
  return uint8_t((u & 0xfeu) | uint8_t(v < 0));
}

float fp8_decode(uint8_t bits, bool is_signed)
{
  uint32_t u = bits;
  if (is_signed) { u &= ~1u; }
  const uint32_t kBase32 = (0x3f800000u | (0x00400000u >> kFp8ValBits)) - (kFp8ExpMask << 23);
  float r                = u2f(kBase32 + (u << (15u + kFp8ExpBits)));
  if (is_signed && (bits & 1u)) { r = -r; }
  return r;
}

uint16_t fp8_decode_half(uint8_t bits, bool is_signed)
{
  uint16_t u = bits;
  if (is_signed) { u &= uint16_t(~1u); }
  const uint16_t kBase16 = uint16_t((0x3c00u | (0x0200u >> kFp8ValBits)) - (kFp8ExpMask << 10));
  uint16_t r             = uint16_t(kBase16 + (u << (2u + kFp8ExpBits)));
  if (is_signed && (bits & 1u)) { r ^= 0x8000u; }
  return r;
}

/* ---------------- dimensions (ivf_pq_index.cu:78-111) ---------------- */

inline uint32_t round_up(uint32_t v, uint32_t m) { return ((v + m - 1) / m) * m; }
inline uint32_t dim_ext_of(uint32_t dim) { return round_up(dim + 1, 8); }
inline uint32_t pq_len_of(uint32_t dim, uint32_t pq_dim) { return (dim + pq_dim - 1) / pq_dim; }

/* ---------------- interleaved list layout ---------------- */

constexpr uint32_t kGroup  = 32;  // kIndexGroupSize   (ivf_pq.hpp:222)
constexpr uint32_t kVecLen = 16;  // kIndexGroupVecLen (ivf_pq.hpp:224)

inline uint32_t codes_per_chunk(uint32_t pq_bits) { return (kVecLen * 8u) / pq_bits; }
inline uint32_t n_chunks_of(uint32_t pq_dim, uint32_t pq_bits)
{
  const uint32_t cpc = codes_per_chunk(pq_bits);
  return (pq_dim + cpc - 1) / cpc;
}

/* address of the 16-byte chunk `m` of row `i` (list extents [groups, chunks, 32, 16],
 * ivf_pq.hpp:288-296; compute_distances_impl.cuh:52-55) */
inline uint64_t chunk_offset(uint32_t i, uint32_t m, uint32_t n_chunks)
{
  return (uint64_t(i / kGroup) * n_chunks + m) * (kGroup * kVecLen) + uint64_t(i % kGroup) * kVecLen;
}

/* code k of a 16-byte little-endian bit stream (ivf_pq_codepacking.cuh:29-75) */
inline uint8_t get_code(const uint8_t* chunk, uint32_t k, uint32_t pq_bits)
{
  const uint32_t bit = k * pq_bits;
  uint32_t pair      = chunk[bit / 8];
  if ((bit % 8) + pq_bits > 8) { pair |= uint32_t(chunk[bit / 8 + 1]) << 8; }
  return uint8_t((pair >> (bit % 8)) & ((1u << pq_bits) - 1u));
}

inline void set_code(uint8_t* chunk, uint32_t k, uint32_t pq_bits, uint8_t code)
{
  const uint32_t bit  = k * pq_bits;
  const uint32_t mask = (1u << pq_bits) - 1u;
  uint32_t pair       = chunk[bit / 8];
  const bool two      = (bit % 8) + pq_bits > 8;
  if (two) { pair |= uint32_t(chunk[bit / 8 + 1]) << 8; }
  pair &= ~(mask << (bit % 8));
  pair |= (uint32_t(code) & mask) << (bit % 8);
  chunk[bit / 8] = uint8_t(pair & 0xffu);
  if (two) { chunk[bit / 8 + 1] = uint8_t(pair >> 8); }
}

inline uint8_t list_code(const uint8_t* list_data, uint32_t row, uint32_t j, uint32_t pq_dim,
                         uint32_t pq_bits)
{
  const uint32_t cpc = codes_per_chunk(pq_bits);
  const uint32_t nch = n_chunks_of(pq_dim, pq_bits);
  return get_code(list_data + chunk_offset(row, j / cpc, nch), j % cpc, pq_bits);
}

/* ---------------- element mapping (detail/ann_utils.cuh:133-201) ---------------- */

inline float map_to_float(const void* rows, int type, uint64_t ix)
{
  switch (type) {
    case ORC_T_F32: return static_cast<const float*>(rows)[ix];
    case ORC_T_F16: return half_to_float(static_cast<const uint16_t*>(rows)[ix]);
    case ORC_T_I8: return float(static_cast<const int8_t*>(rows)[ix]) * (1.0f / 128.0f);
    case ORC_T_U8: return float(static_cast<const uint8_t*>(rows)[ix]) * (1.0f / 256.0f);
    default: return 0.0f;
  }
}

inline float scaling_factor(int type)
{
  // utils::config<T>::kDivisor / utils::config<float>::kDivisor  (ivf_pq_search.cuh:1043)
  return type == ORC_T_U8 ? 256.0f : (type == ORC_T_I8 ? 128.0f : 1.0f);
}

inline bool is_ip_like(int metric)
{
  return metric == ORC_InnerProduct || metric == ORC_CosineExpanded;
}

/* ---------------- coarse search (ivf_pq_search.cuh:60-168) ---------------- */

/* score of every list for one mapped query.  The reference evaluates a GEMM over dim_ext columns
 * where query column `dim` is -0.5 (L2) or 0 (IP/cosine) and the remaining padding is zero, then
 * scales by alpha = -2 (L2) or -1.  Accumulation: fp32 FMA, columns ascending. */
void coarse_scores_f32(const orc_index& ix, const float* qf, float* scores)
{
  const uint32_t de  = dim_ext_of(ix.dim);
  const bool ip      = is_ip_like(ix.metric);
  const float qnorm  = ip ? 0.0f : -0.5f;
  const float alpha  = ip ? -1.0f : -2.0f;
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    const float* c = ix.centers + uint64_t(l) * de;
    float acc      = 0.0f;
    for (uint32_t d = 0; d < ix.dim; d++) { acc = std::fmaf(c[d], qf[d], acc); }
    acc       = std::fmaf(c[ix.dim], qnorm, acc);
    scores[l] = alpha * acc;
  }
}

/* half-precision variant (ivf_pq_search.cuh:258-340): centres and queries rounded to binary16,
 * products accumulated in fp32 (FMA, ascending), result rounded to binary16 after scaling.
 * The arithmetic stated here is pinned by tests/test_oracle_search.py (numpy float16); that the
 * reference's half GEMM accumulates this way is a cuBLAS detail: parity unpinned for the
 * accumulation type. */
void coarse_scores_f16(const orc_index& ix, const float* qf, float* scores)
{
  const uint32_t de = dim_ext_of(ix.dim);
  const bool ip     = is_ip_like(ix.metric);
  const float qnorm = ip ? 0.0f : -0.5f;
  const float alpha = ip ? -1.0f : -2.0f;
  std::vector<float> qh(ix.dim);
  for (uint32_t d = 0; d < ix.dim; d++) { qh[d] = half_to_float(float_to_half(qf[d])); }
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    const float* c = ix.centers + uint64_t(l) * de;
    float acc      = 0.0f;
    for (uint32_t d = 0; d < ix.dim; d++) {
      acc = std::fmaf(half_to_float(float_to_half(c[d])), qh[d], acc);
    }
    acc       = std::fmaf(half_to_float(float_to_half(c[ix.dim])), qnorm, acc);
    scores[l] = half_to_float(float_to_half(alpha * acc));
  }
}

/* 8-bit integer variant (ivf_pq_search.cuh:170-256; centres quantised as in
 * cpp/src/neighbors/ivf_pq_index.cu:661-738).  Rows have dim_ext_int8 = round_up(dim + 2, 16)
 * columns.  Centre side: column c < dim is trunc(clamp(128 c)); the squared norm x is split as
 * y = clamp(x * 64 / (m - 1)), m = dim_ext_int8 - dim: every column past `dim` holds round(y) and
 * column `dim` holds trunc(clamp(128 (y - round(y)))).  Query side: mapping<int8_t> of the element
 * (trunc(clamp(128 q)) for float types, x >> 1 for uint8, x for int8), column `dim` holds 1 - m,
 * the columns past it -128 (L2) or 0 (inner product, cosine).  Scores are int32: alpha times the
 * dot product, alpha = -2 (L2) or -1.
 *
 * Both operands have dim_ext_int8 columns in the reference as well: its driver takes the row
 * length of the int8 centre matrix as `dim_ext` whenever coarse_search_dtype is CUDA_R_8I
 * (ivf_pq_search.cuh:929-931), and select_clusters pads the query rows to it. */
inline uint32_t dim_ext_int8_of(uint32_t dim) { return round_up(dim + 2, 16); }

inline int8_t clamp_to_int8(float v)
{
  // static_cast<int8_t>(fmaxf(-128, fminf(127, v))): truncation toward zero
  return int8_t(std::fmax(-128.0f, std::fmin(127.0f, v)));
}

void center_row_int8(const orc_index& ix, uint32_t l, int8_t* out)
{
  const uint32_t de  = dim_ext_of(ix.dim);
  const uint32_t de8 = dim_ext_int8_of(ix.dim);
  const float* c     = ix.centers + uint64_t(l) * de;
  for (uint32_t d = 0; d < ix.dim; d++) { out[d] = clamp_to_int8(c[d] * 128.0f); }
  const float x = c[ix.dim];
  const float f = 64.0f / float(de8 - ix.dim - 1);
  const float y = std::fmax(-128.0f, std::fmin(127.0f, x * f));
  const float z = std::fmax(-128.0f, std::fmin(127.0f, (y - std::round(y)) * 128.0f));
  out[ix.dim]   = int8_t(z);
  for (uint32_t d = ix.dim + 1; d < de8; d++) { out[d] = int8_t(std::round(y)); }
}

void query_row_int8(const orc_index& ix, const float* qf, int8_t* out)
{
  const uint32_t de8 = dim_ext_int8_of(ix.dim);
  const int m        = int(de8 - ix.dim);
  const int8_t nf    = is_ip_like(ix.metric) ? int8_t(0) : int8_t(-128);
  // qf = mapping<float>(element): x / 256 (uint8), x / 128 (int8): 128 qf gives x / 2 and x, and
  // truncation gives mapping<int8_t>'s x >> 1 and x
  for (uint32_t d = 0; d < ix.dim; d++) { out[d] = clamp_to_int8(qf[d] * 128.0f); }
  out[ix.dim] = int8_t(1 - m);
  for (uint32_t d = ix.dim + 1; d < de8; d++) { out[d] = nf; }
}

void coarse_scores_i8(const orc_index& ix, const float* qf, int32_t* scores)
{
  const uint32_t de8  = dim_ext_int8_of(ix.dim);
  const int32_t alpha = is_ip_like(ix.metric) ? -1 : -2;
  std::vector<int8_t> q8(de8), c8(de8);
  query_row_int8(ix, qf, q8.data());
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    center_row_int8(ix, l, c8.data());
    int32_t acc = 0;
    for (uint32_t d = 0; d < de8; d++) { acc += int32_t(c8[d]) * int32_t(q8[d]); }
    scores[l] = alpha * acc;
  }
}

/* total order used by every selection in this file: smaller score first, then smaller index.
 * -0.0 and +0.0 compare equal, as they do on the device. */
struct cand {
  float score;
  uint32_t id;
};
inline bool cand_less(const cand& a, const cand& b)
{
  return a.score < b.score || (a.score == b.score && a.id < b.id);
}

void select_smallest(std::vector<cand>& v, uint32_t k)
{
  if (v.size() > k) {
    std::nth_element(v.begin(), v.begin() + k, v.end(), cand_less);
    v.resize(k);
  }
  std::sort(v.begin(), v.end(), cand_less);
}

void map_query(const orc_index& ix, const void* queries, int type, uint64_t q, float* qf)
{
  for (uint32_t d = 0; d < ix.dim; d++) { qf[d] = map_to_float(queries, type, q * ix.dim + d); }
}

void select_clusters_one(const orc_index& ix, const orc_search_params& sp, const float* qf,
                         uint32_t n_probes, std::vector<float>& scores, std::vector<cand>& tmp,
                         uint32_t* probes, float* probe_scores)
{
  if (sp.coarse_search_dtype == ORC_R_8I) {
    std::vector<int32_t> si(ix.n_lists);
    coarse_scores_i8(ix, qf, si.data());
    std::vector<std::pair<int32_t, uint32_t>> order(ix.n_lists);
    for (uint32_t l = 0; l < ix.n_lists; l++) { order[l] = {si[l], l}; }
    std::partial_sort(order.begin(), order.begin() + n_probes, order.end());
    for (uint32_t p = 0; p < n_probes; p++) {
      probes[p] = order[p].second;
      if (probe_scores) { probe_scores[p] = float(order[p].first); }
    }
    return;
  }
  scores.resize(ix.n_lists);
  if (sp.coarse_search_dtype == ORC_R_16F) {
    coarse_scores_f16(ix, qf, scores.data());
  } else {
    coarse_scores_f32(ix, qf, scores.data());
  }
  tmp.resize(ix.n_lists);
  for (uint32_t l = 0; l < ix.n_lists; l++) { tmp[l] = cand{scores[l], l}; }
  select_smallest(tmp, n_probes);
  for (uint32_t p = 0; p < n_probes; p++) {
    probes[p] = tmp[p].id;
    if (probe_scores) { probe_scores[p] = tmp[p].score; }
  }
}

/* ---------------- query rotation (ivf_pq_search.cuh:996-1025) ---------------- */

/* The rotation GEMM takes the query rows the coarse search made and the rotation matrix in the
 * same type (get_rotation_matrix<value_type>, ivf_pq_search.cuh:996-1019): fp32; binary16 copies of
 * both (products accumulated in fp32 here, result fp32); or int8 copies (mapping<int8_t>: 128 x
 * clamped and truncated) with the integer dot product scaled by 1 / 128^2. */
void rotate_query(const orc_index& ix, int coarse_dtype, const float* qf, float* rq)
{
  const uint32_t rot_dim = pq_len_of(ix.dim, ix.pq_dim) * ix.pq_dim;
  for (uint32_t r = 0; r < rot_dim; r++) {
    const float* row = ix.rotation_matrix + uint64_t(r) * ix.dim;
    if (coarse_dtype == ORC_R_8I) {
      int32_t acc = 0;
      for (uint32_t d = 0; d < ix.dim; d++) {
        acc += int32_t(clamp_to_int8(row[d] * 128.0f)) * int32_t(clamp_to_int8(qf[d] * 128.0f));
      }
      rq[r] = float(acc) * (1.0f / 128.0f / 128.0f);
      continue;
    }
    float acc = 0.0f;
    if (coarse_dtype == ORC_R_16F) {
      for (uint32_t d = 0; d < ix.dim; d++) {
        acc = std::fmaf(half_to_float(float_to_half(row[d])), half_to_float(float_to_half(qf[d])), acc);
      }
    } else {
      for (uint32_t d = 0; d < ix.dim; d++) { acc = std::fmaf(row[d], qf[d], acc); }
    }
    rq[r] = acc;
  }
  if (ix.metric == ORC_CosineExpanded) {
    // row_normalize<L2Norm>: divide by sqrt(sum of squares); sum accumulates ascending with FMA
    float ss = 0.0f;
    for (uint32_t r = 0; r < rot_dim; r++) { ss = std::fmaf(rq[r], rq[r], ss); }
    const float nrm = std::sqrt(ss);
    if (nrm > 0.0f) {
      for (uint32_t r = 0; r < rot_dim; r++) { rq[r] = rq[r] / nrm; }
    }
  }
}

/* ---------------- lookup table (create_lut_impl.cuh:16-79) ---------------- */

/* fp32 table of one (query, list) pair before rounding to the LUT type.
 * L2:  score = sum_t ((rq - c_rot) - book)^2, `+= d*d` as one FMA.
 * IP:  the reference's preferred variant stages (q, q*c_rot) per dimension
 *      (precompute_base_diff_impl.cuh:28-41) and then does `score -= q*c; score -= q * book`,
 *      the latter contracted to an FMA. */
void make_lut_f32(const orc_index& ix, const float* rq, uint32_t label, float* lut)
{
  const uint32_t pq_len  = pq_len_of(ix.dim, ix.pq_dim);
  const uint32_t rot_dim = pq_len * ix.pq_dim;
  const uint32_t B       = 1u << ix.pq_bits;
  const float* c_rot     = ix.centers_rot + uint64_t(label) * rot_dim;
  const bool ip          = is_ip_like(ix.metric);
  for (uint32_t j = 0; j < ix.pq_dim; j++) {
    const float* book = ix.pq_centers + uint64_t(pq_len) * B *
                                          (ix.codebook_kind == ORC_PER_SUBSPACE ? j : label);
    for (uint32_t code = 0; code < B; code++) {
      float score = 0.0f;
      for (uint32_t t = 0; t < pq_len; t++) {
        const uint32_t d = j * pq_len + t;
        const float pqc  = book[uint64_t(t) * B + code];
        if (!ip) {
          float diff = rq[d] - c_rot[d];
          diff -= pqc;
          score = std::fmaf(diff, diff, score);
        } else {
          const float q  = rq[d];
          const float qc = c_rot[d] * q;
          score -= qc;
          score = std::fmaf(-q, pqc, score);
        }
      }
      lut[uint64_t(j) * B + code] = score;
    }
  }
}

enum lut_kind { LUT_F32, LUT_F16, LUT_FP8U, LUT_FP8S };

lut_kind lut_kind_of(const orc_index& ix, const orc_search_params& sp)
{
  // ivf_pq_search.cuh:709-729
  if (sp.lut_dtype == ORC_R_32F) return LUT_F32;
  if (sp.lut_dtype == ORC_R_16F) return LUT_F16;
  return is_ip_like(ix.metric) ? LUT_FP8S : LUT_FP8U;
}

/* ---------------- scan of one list (compute_distances_impl.cuh:73-90,
 *                  compute_score_impl.cuh:13-79) ---------------- */

/* Rounded LUT entries are kept in the accumulation type: for OutT=float as floats, for OutT=half
 * as half bit patterns.  `score = OutT(score + OutT(LUT[j][code]))`, j ascending. */
struct pair_lut {
  std::vector<float> f32;   // OutT(LutT(x)) when OutT is float
  std::vector<uint16_t> h;  // OutT(LutT(x)) when OutT is half
};

void round_lut(const std::vector<float>& raw, lut_kind kind, bool out_half, pair_lut& out)
{
  const size_t n = raw.size();
  if (out_half) {
    out.h.resize(n);
  } else {
    out.f32.resize(n);
  }
  for (size_t i = 0; i < n; i++) {
    switch (kind) {
      case LUT_F32: out.f32[i] = raw[i]; break;  // (half, float) is rejected earlier
      case LUT_F16: {
        const uint16_t h = float_to_half(raw[i]);
        if (out_half) {
          out.h[i] = h;
        } else {
          out.f32[i] = half_to_float(h);
        }
      } break;
      case LUT_FP8U:
      case LUT_FP8S: {
        const bool sg   = kind == LUT_FP8S;
        const uint8_t u = fp8_encode(raw[i], sg);
        if (out_half) {
          out.h[i] = fp8_decode_half(u, sg);
        } else {
          out.f32[i] = fp8_decode(u, sg);
        }
      } break;
    }
  }
}

/* ---------------- post-processing (ivf_common.cuh:175-252) ---------------- */

float postprocess_distance(float d, int metric, float s)
{
  switch (metric) {
    case ORC_L2Expanded: return s != 1.0f ? d * (s * s) : d;
    case ORC_L2SqrtExpanded: return s != 1.0f ? std::sqrt(d) * s : std::sqrt(d);
    case ORC_InnerProduct: return d * (-1.0f * s * s);
    case ORC_CosineExpanded: return s != 1.0f ? d * (s * s) : d;
    default: return d;
  }
}

template <typename F>
void parallel_for(uint64_t n, int n_threads, F&& body)
{
  if (n_threads <= 1 || n <= 1) {
    for (uint64_t i = 0; i < n; i++) { body(i, 0); }
    return;
  }
  std::atomic<uint64_t> next{0};
  std::vector<std::thread> pool;
  for (int t = 0; t < n_threads; t++) {
    pool.emplace_back([&, t] {
      for (;;) {
        const uint64_t i = next.fetch_add(1);
        if (i >= n) { break; }
        body(i, t);
      }
    });
  }
  for (auto& th : pool) { th.join(); }
}

bool validate(const orc_index& ix, const orc_search_params& sp, uint32_t k, bool for_search)
{
  // ivf_pq_search.cuh:901-923 and ivf_pq_index.cu:599-609
  if (ix.pq_bits < 4 || ix.pq_bits > 8) {
    g_error = "pq_bits must be within [4, 8]";
    return false;
  }
  if ((ix.pq_bits * ix.pq_dim) % 8 != 0) {
    g_error = "pq_bits * pq_dim must be a multiple of 8";
    return false;
  }
  if (sp.internal_distance_dtype != ORC_R_16F && sp.internal_distance_dtype != ORC_R_32F) {
    g_error = "internal_distance_dtype must be either CUDA_R_16F or CUDA_R_32F";
    return false;
  }
  if (sp.lut_dtype != ORC_R_16F && sp.lut_dtype != ORC_R_32F && sp.lut_dtype != ORC_R_8U) {
    g_error = "lut_dtype must be CUDA_R_16F, CUDA_R_32F or CUDA_R_8U";
    return false;
  }
  if (sp.internal_distance_dtype == ORC_R_16F && sp.lut_dtype == ORC_R_32F) {
    g_error = "Unexpected lut_dtype / internal_distance_dtype combination";
    return false;
  }
  if (sp.coarse_search_dtype != ORC_R_32F && sp.coarse_search_dtype != ORC_R_16F &&
      sp.coarse_search_dtype != ORC_R_8I) {
    g_error = "Unsupported coarse_search_dtype in the oracle";
    return false;
  }
  if (sp.n_probes == 0) {
    g_error = "n_probes (number of clusters to probe in the search) must be positive.";
    return false;
  }
  if (for_search) {
    if (k == 0) {
      g_error = "parameter `k` in top-k must be positive.";
      return false;
    }
    uint64_t size = 0;
    for (uint32_t l = 0; l < ix.n_lists; l++) { size += ix.list_sizes[l]; }
    if (k > size) {
      g_error = "parameter `k` in top-k must not be larger that the total size of the index";
      return false;
    }
  }
  return true;
}

}  // namespace

extern "C" {

/* ---------------- refinement (refine_device.cuh:35-135) ---------------- */

int orc_refine(const void* dataset, const void* queries, int row_type, int64_t n_rows,
               uint32_t n_queries, uint32_t dim, const int64_t* candidates, uint32_t n_candidates,
               uint32_t k, int metric, int64_t* indices, float* distances)
{
  if (k == 0 || k > n_candidates) {
    g_error = "refine: k must be within [1, n_candidates]";
    return 1;
  }
  if (metric != ORC_L2Expanded && metric != ORC_L2SqrtExpanded && metric != ORC_InnerProduct) {
    g_error = "refine: unsupported metric";
    return 1;
  }
  const bool ip = metric == ORC_InnerProduct;
  struct scored {
    float ordered;  // smaller is better
    uint32_t slot;
  };
  std::vector<scored> v;
  for (uint32_t q = 0; q < n_queries; q++) {
    v.clear();
    for (uint32_t c = 0; c < n_candidates; c++) {
      const int64_t id = candidates[uint64_t(q) * n_candidates + c];
      if (id < 0 || id >= n_rows) { continue; }
      float dist = 0.0f;
      if (row_type == ORC_T_F32 || row_type == ORC_T_F16) {
        float acc = 0.0f;
        for (uint32_t d = 0; d < dim; d++) {
          float a, b;
          if (row_type == ORC_T_F32) {
            a = static_cast<const float*>(queries)[uint64_t(q) * dim + d];
            b = static_cast<const float*>(dataset)[uint64_t(id) * dim + d];
          } else {
            a = half_to_float(static_cast<const uint16_t*>(queries)[uint64_t(q) * dim + d]);
            b = half_to_float(static_cast<const uint16_t*>(dataset)[uint64_t(id) * dim + d]);
          }
          if (ip) {
            acc += a * b;
          } else {
            const float diff = a - b;
            acc += diff * diff;
          }
        }
        dist = acc;
      } else {
        int64_t acc = 0;  // exact; the reference's 32-bit accumulators hold these sums too
        for (uint32_t d = 0; d < dim; d++) {
          int32_t a, b;
          if (row_type == ORC_T_I8) {
            a = static_cast<const int8_t*>(queries)[uint64_t(q) * dim + d];
            b = static_cast<const int8_t*>(dataset)[uint64_t(id) * dim + d];
          } else {
            a = static_cast<const uint8_t*>(queries)[uint64_t(q) * dim + d];
            b = static_cast<const uint8_t*>(dataset)[uint64_t(id) * dim + d];
          }
          acc += ip ? int64_t(a) * b : int64_t(a - b) * (a - b);
        }
        dist = row_type == ORC_T_I8 ? float(int32_t(acc)) : float(uint32_t(acc));
      }
      v.push_back(scored{ip ? -dist : dist, c});
    }
    std::sort(v.begin(), v.end(), [](const scored& x, const scored& y) {
      return x.ordered < y.ordered || (x.ordered == y.ordered && x.slot < y.slot);
    });
    for (uint32_t r = 0; r < k; r++) {
      int64_t id = -1;
      float d    = FLT_MAX;
      if (r < v.size()) {
        id = candidates[uint64_t(q) * n_candidates + v[r].slot];
        d  = ip ? -v[r].ordered : v[r].ordered;
        if (metric == ORC_L2SqrtExpanded) { d = std::sqrt(d); }
      }
      indices[uint64_t(q) * k + r]   = id;
      distances[uint64_t(q) * k + r] = d;
    }
  }
  return 0;
}

const char* orc_last_error(void) { return g_error.c_str(); }

uint32_t orc_dim_ext(uint32_t dim) { return dim_ext_of(dim); }
uint32_t orc_pq_len(uint32_t dim, uint32_t pq_dim) { return pq_len_of(dim, pq_dim); }
uint32_t orc_rot_dim(uint32_t dim, uint32_t pq_dim) { return pq_len_of(dim, pq_dim) * pq_dim; }

uint16_t orc_float_to_half(float v) { return float_to_half(v); }
float orc_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t orc_half_add(uint16_t a, uint16_t b) { return half_add(a, b); }
uint8_t orc_fp8_encode(float v, int is_signed) { return fp8_encode(v, is_signed != 0); }
float orc_fp8_decode(uint8_t u, int is_signed) { return fp8_decode(u, is_signed != 0); }
uint16_t orc_fp8_decode_half(uint8_t u, int is_signed) { return fp8_decode_half(u, is_signed != 0); }

uint64_t orc_list_bytes(uint32_t n_rows, uint32_t pq_dim, uint32_t pq_bits)
{
  return uint64_t(round_up(n_rows, kGroup) / kGroup) * n_chunks_of(pq_dim, pq_bits) * kGroup *
         kVecLen;
}

void orc_pack_list(const uint8_t* codes, uint32_t n_rows, uint32_t pq_dim, uint32_t pq_bits,
                   uint32_t row_offset, uint8_t* list_data)
{
  const uint32_t cpc = codes_per_chunk(pq_bits);
  const uint32_t nch = n_chunks_of(pq_dim, pq_bits);
  for (uint32_t r = 0; r < n_rows; r++) {
    for (uint32_t m = 0; m < nch; m++) {
      uint8_t* chunk = list_data + chunk_offset(row_offset + r, m, nch);
      std::memset(chunk, 0, kVecLen);  // write_vector_interleaved clears each chunk first
      for (uint32_t k = 0; k < cpc && m * cpc + k < pq_dim; k++) {
        set_code(chunk, k, pq_bits, codes[uint64_t(r) * pq_dim + m * cpc + k]);
      }
    }
  }
}

void orc_unpack_list(const uint8_t* list_data, uint32_t n_rows, uint32_t pq_dim, uint32_t pq_bits,
                     uint32_t row_offset, uint8_t* codes)
{
  for (uint32_t r = 0; r < n_rows; r++) {
    for (uint32_t j = 0; j < pq_dim; j++) {
      codes[uint64_t(r) * pq_dim + j] = list_code(list_data, row_offset + r, j, pq_dim, pq_bits);
    }
  }
}

void orc_unpack_list_contiguous(const uint8_t* list_data, uint32_t n_rows, uint32_t pq_dim,
                                uint32_t pq_bits, uint32_t row_offset, uint8_t* out)
{
  // unpack_contiguous_list_data: codes of one row form a single little-endian bit stream
  const uint32_t row_bytes = (pq_dim * pq_bits + 7) / 8;
  std::memset(out, 0, uint64_t(n_rows) * row_bytes);
  for (uint32_t r = 0; r < n_rows; r++) {
    uint8_t* row = out + uint64_t(r) * row_bytes;
    for (uint32_t j = 0; j < pq_dim; j++) {
      const uint32_t code = list_code(list_data, row_offset + r, j, pq_dim, pq_bits);
      const uint32_t bit  = j * pq_bits;
      row[bit / 8] |= uint8_t(code << (bit % 8));
      if ((bit % 8) + pq_bits > 8) { row[bit / 8 + 1] |= uint8_t(code >> (8 - bit % 8)); }
    }
  }
}

int orc_select_clusters(const orc_index* index, const orc_search_params* params,
                        const void* queries, int query_type, uint32_t n_queries, uint32_t* probes,
                        float* probe_scores, int n_threads)
{
  if (!validate(*index, *params, 1, false)) { return 1; }
  const uint32_t P = std::min(params->n_probes, index->n_lists);
  struct scratch {
    std::vector<float> qf, scores;
    std::vector<cand> tmp;
  };
  std::vector<scratch> sc(std::max(n_threads, 1));
  parallel_for(n_queries, n_threads, [&](uint64_t q, int t) {
    auto& s = sc[t];
    s.qf.resize(index->dim);
    map_query(*index, queries, query_type, q, s.qf.data());
    select_clusters_one(*index, *params, s.qf.data(), P, s.scores, s.tmp, probes + q * P,
                        probe_scores ? probe_scores + q * P : nullptr);
  });
  return 0;
}

int orc_make_lut(const orc_index* index, const orc_search_params* params, const void* query,
                 int query_type, uint32_t label, void* lut_out)
{
  if (!validate(*index, *params, 1, false)) { return 1; }
  const orc_index& ix = *index;
  const uint32_t rot  = orc_rot_dim(ix.dim, ix.pq_dim);
  std::vector<float> qf(ix.dim), rq(rot), raw(uint64_t(ix.pq_dim) << ix.pq_bits);
  map_query(ix, query, query_type, 0, qf.data());
  rotate_query(ix, params->coarse_search_dtype, qf.data(), rq.data());
  make_lut_f32(ix, rq.data(), label, raw.data());
  const lut_kind kind = lut_kind_of(ix, *params);
  for (size_t i = 0; i < raw.size(); i++) {
    switch (kind) {
      case LUT_F32: static_cast<float*>(lut_out)[i] = raw[i]; break;
      case LUT_F16: static_cast<uint16_t*>(lut_out)[i] = float_to_half(raw[i]); break;
      case LUT_FP8U: static_cast<uint8_t*>(lut_out)[i] = fp8_encode(raw[i], false); break;
      case LUT_FP8S: static_cast<uint8_t*>(lut_out)[i] = fp8_encode(raw[i], true); break;
    }
  }
  return 0;
}

int orc_search(const orc_index* index, const orc_search_params* params, const void* queries,
               int query_type, uint32_t n_queries, uint32_t k, const uint32_t* filter_bitset,
               int64_t filter_nbits, int64_t* neighbors, float* distances, uint32_t* probes_out,
               int n_threads)
{
  if (!validate(*index, *params, k, true)) { return 1; }
  const orc_index& ix    = *index;
  const uint32_t P       = std::min(params->n_probes, ix.n_lists);
  const uint32_t rot     = orc_rot_dim(ix.dim, ix.pq_dim);
  const uint32_t B       = 1u << ix.pq_bits;
  const lut_kind kind    = lut_kind_of(ix, *params);
  const bool out_half    = params->internal_distance_dtype == ORC_R_16F;
  const bool cosine      = ix.metric == ORC_CosineExpanded;
  const float s          = scaling_factor(query_type);
  const uint32_t cpc     = codes_per_chunk(ix.pq_bits);
  const uint32_t nch     = n_chunks_of(ix.pq_dim, ix.pq_bits);
  const uint16_t one_h   = 0x3c00u;

  struct scratch {
    std::vector<float> qf, rq, scores, raw;
    std::vector<cand> tmp, best;
    std::vector<uint32_t> probes, chunk;
    pair_lut lut;
  };
  std::vector<scratch> sc(std::max(n_threads, 1));

  parallel_for(n_queries, n_threads, [&](uint64_t q, int t) {
    auto& w = sc[t];
    w.qf.resize(ix.dim);
    w.rq.resize(rot);
    w.probes.resize(P);
    w.chunk.resize(P);
    w.raw.resize(uint64_t(ix.pq_dim) * B);
    map_query(ix, queries, query_type, q, w.qf.data());
    select_clusters_one(ix, *params, w.qf.data(), P, w.scores, w.tmp, w.probes.data(), nullptr);
    if (probes_out) { std::memcpy(probes_out + q * P, w.probes.data(), P * sizeof(uint32_t)); }
    rotate_query(ix, params->coarse_search_dtype, w.qf.data(), w.rq.data());

    // calc_chunk_indices (ivf_common.cu:21-50): inclusive prefix sums of probed list sizes
    uint32_t total = 0;
    for (uint32_t p = 0; p < P; p++) {
      total += ix.list_sizes[w.probes[p]];
      w.chunk[p] = total;
    }

    w.best.clear();
    for (uint32_t p = 0; p < P; p++) {
      const uint32_t label      = w.probes[p];
      const uint32_t n_rows     = ix.list_sizes[label];
      const uint32_t sample_off = p ? w.chunk[p - 1] : 0;
      if (n_rows == 0) { continue; }
      make_lut_f32(ix, w.rq.data(), label, w.raw.data());
      round_lut(w.raw, kind, out_half, w.lut);
      const uint8_t* data = ix.list_data[label];
      const int64_t* inds = ix.list_inds[label];
      for (uint32_t i = 0; i < n_rows; i++) {
        if (filter_bitset != nullptr) {
          // bitset_filter over source ids: set bit == keep (sample_filter.cuh:94-101)
          const int64_t id = inds[i];
          if (id < 0 || id >= filter_nbits) { continue; }
          if (((filter_bitset[id >> 5] >> (id & 31)) & 1u) == 0) { continue; }
        }
        float score_f;
        if (!out_half) {
          float acc = 0.0f;
          for (uint32_t j = 0; j < ix.pq_dim; j++) {
            const uint8_t code = get_code(data + chunk_offset(i, j / cpc, nch), j % cpc, ix.pq_bits);
            acc += w.lut.f32[uint64_t(j) * B + code];
          }
          if (cosine) { acc += 1.0f; }  // increment_score_impl.cuh:12-18
          score_f = acc;
        } else {
          uint16_t acc = 0;
          for (uint32_t j = 0; j < ix.pq_dim; j++) {
            const uint8_t code = get_code(data + chunk_offset(i, j / cpc, nch), j % cpc, ix.pq_bits);
            acc = half_add(acc, w.lut.h[uint64_t(j) * B + code]);
          }
          if (cosine) { acc = half_add(acc, one_h); }
          score_f = half_to_float(acc);
        }
        if (std::isnan(score_f)) { continue; }  // a NaN never wins a `<` comparison on the device
        w.best.push_back(cand{score_f, sample_off + i});
        if (w.best.size() >= size_t(k) * 4 + 4096) { select_smallest(w.best, k); }
      }
    }
    select_smallest(w.best, k);

    for (uint32_t r = 0; r < k; r++) {
      int64_t id = std::numeric_limits<int64_t>::max();  // kOutOfBoundsRecord (ivf_common.cuh:30)
      float d    = std::numeric_limits<float>::max();    // dummy score of an unfilled slot
      if (r < w.best.size()) {
        // find_chunk_ix (ivf_common.cuh:94-110): first probe whose inclusive end exceeds the sample
        const uint32_t sample = w.best[r].id;
        const uint32_t slot =
          uint32_t(std::upper_bound(w.chunk.begin(), w.chunk.end(), sample) - w.chunk.begin());
        const uint32_t off = sample - (slot ? w.chunk[slot - 1] : 0);
        id                 = ix.list_inds[w.probes[slot]][off];
        d                  = w.best[r].score;
      }
      neighbors[q * k + r] = id;
      distances[q * k + r] = postprocess_distance(d, ix.metric, s);
    }
  });
  return 0;
}

int orc_encode(const orc_index* index, const void* rows, int row_type, uint64_t n_rows,
               uint32_t* labels, uint8_t* codes, int n_threads)
{
  const orc_index& ix   = *index;
  const uint32_t pq_len = pq_len_of(ix.dim, ix.pq_dim);
  const uint32_t rot    = pq_len * ix.pq_dim;
  const uint32_t B      = 1u << ix.pq_bits;
  const uint32_t de     = dim_ext_of(ix.dim);
  orc_search_params sp{1, ORC_R_32F, ORC_R_32F, ORC_R_32F};
  orc_index ix_labels = ix;
  if (ix.metric == ORC_InnerProduct) { ix_labels.metric = ORC_L2Expanded; }
  struct scratch {
    std::vector<float> xf, diff, res, scores;
    std::vector<cand> tmp;
  };
  std::vector<scratch> sc(std::max(n_threads, 1));
  parallel_for(n_rows, n_threads, [&](uint64_t r, int t) {
    auto& w = sc[t];
    w.xf.resize(ix.dim);
    w.diff.resize(ix.dim);
    w.res.resize(rot);
    map_query(ix, rows, row_type, r, w.xf.data());
    if (ix.metric == ORC_CosineExpanded) {
      float ss = 0.0f;
      for (uint32_t d = 0; d < ix.dim; d++) { ss = std::fmaf(w.xf[d], w.xf[d], ss); }
      const float nrm = std::sqrt(ss);
      if (nrm > 0.0f) {
        for (uint32_t d = 0; d < ix.dim; d++) { w.xf[d] = w.xf[d] / nrm; }
      }
    }
    // the list is chosen with the coarse clustering's metric: L2 also for an inner-product index
    // (coarse_clustering_metric, ivf_pq_build.cuh:70-76, :1141; ivf_pq_transform.cuh:58)
    uint32_t label;
    select_clusters_one(ix_labels, sp, w.xf.data(), 1, w.scores, w.tmp, &label, nullptr);
    labels[r] = label;
    // residual = rotation_matrix * (x - centre[label])   (ivf_pq_build.cuh:140-206)
    const float* c = ix.centers + uint64_t(label) * de;
    for (uint32_t d = 0; d < ix.dim; d++) { w.diff[d] = w.xf[d] - c[d]; }
    for (uint32_t o = 0; o < rot; o++) {
      const float* row = ix.rotation_matrix + uint64_t(o) * ix.dim;
      float acc        = 0.0f;
      for (uint32_t d = 0; d < ix.dim; d++) { acc = std::fmaf(row[d], w.diff[d], acc); }
      w.res[o] = acc;
    }
    // nearest codebook entry per subspace, lowest code wins ties
    // (ivf_pq_process_and_fill_codes.cuh:84-126)
    for (uint32_t j = 0; j < ix.pq_dim; j++) {
      const float* book = ix.pq_centers + uint64_t(pq_len) * B *
                                            (ix.codebook_kind == ORC_PER_SUBSPACE ? j : label);
      float best   = std::numeric_limits<float>::infinity();
      uint8_t code = 0;
      for (uint32_t l = 0; l < B; l++) {
        float d = 0.0f;
        for (uint32_t tt = 0; tt < pq_len; tt++) {
          const float v = w.res[j * pq_len + tt] - book[uint64_t(tt) * B + l];
          d             = std::fmaf(v, v, d);
        }
        if (d < best) {
          best = d;
          code = uint8_t(l);
        }
      }
      codes[r * ix.pq_dim + j] = code;
    }
  });
  return 0;
}

}  // extern "C"
