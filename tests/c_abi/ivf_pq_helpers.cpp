/*
 * A C++17 caller of ivf_pq::helpers (reading and editing single lists), compiled by the host
 * compiler alone.  The checks are those of the reference's own tests of these helpers
 * (cpp/tests/neighbors/ann_ivf_pq.cuh:316-470: check_reconstruction, check_reconstruct_extend,
 * check_packing) plus closed forms computed here on the host: the bit-contiguous form of a row
 * (code j at bit j * pq_bits, least significant first) and the decoded vector
 * rotation^T (rotated centre + codebook entries) in double precision from the model tensors.
 * Runs 4- to 8-bit codes, rows of one and of two chunks, per-subspace and per-cluster codebooks.
 * Prints "ok".
 */
#include <cuvs/neighbors/ivf_pq.hpp>

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

namespace {

#define REQUIRE(cond)                                                     \
  do {                                                                    \
    if (!(cond)) {                                                        \
      std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
      std::exit(1);                                                       \
    }                                                                     \
  } while (0)

template <typename T>
T* device_array(size_t n)
{
  void* ptr = nullptr;
  REQUIRE(hipMalloc(&ptr, std::max<size_t>(n, 1) * sizeof(T)) == hipSuccess);
  return static_cast<T*>(ptr);
}

template <typename T>
T* to_device(const std::vector<T>& host)
{
  T* ptr = device_array<T>(host.size());
  REQUIRE(hipMemcpy(ptr, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) == hipSuccess);
  return ptr;
}

template <typename T>
std::vector<T> to_host(const T* device, size_t n)
{
  std::vector<T> host(n);
  if (n > 0) { REQUIRE(hipMemcpy(host.data(), device, n * sizeof(T), hipMemcpyDeviceToHost) == hipSuccess); }
  return host;
}

using namespace cuvs::neighbors;
using cuvs::make_device_matrix_view;
using cuvs::make_device_vector_view;
namespace packer = ivf_pq::helpers::codepacker;

struct list_snapshot {
  uint32_t size = 0;
  std::vector<uint8_t> bytes;  // the list's interleaved groups
  std::vector<int64_t> ids;
};

list_snapshot snapshot(const ivf_pq::index<int64_t>& index, uint32_t label)
{
  list_snapshot s;
  s.size                  = to_host(index.list_sizes(), index.n_lists())[label];
  const uint32_t per      = 128 / index.pq_bits();
  const uint32_t n_chunks = (index.pq_dim() + per - 1) / per;
  const auto data_ptrs    = to_host(index.data_ptrs(), index.n_lists());
  const auto inds_ptrs    = to_host(index.inds_ptrs(), index.n_lists());
  s.bytes                 = to_host(data_ptrs[label], size_t((s.size + 31) / 32) * n_chunks * 512);
  s.ids                   = to_host(inds_ptrs[label], s.size);
  return s;
}

/** Closed form of a bit-contiguous row: code j occupies bits [j * bits, (j + 1) * bits). */
std::vector<uint8_t> contiguous_rows(const std::vector<uint8_t>& codes, size_t n, uint32_t pq_dim, uint32_t bits)
{
  const size_t row_bytes = (pq_dim * bits + 7) / 8;
  std::vector<uint8_t> out(n * row_bytes, 0);
  for (size_t i = 0; i < n; i++) {
    for (uint32_t j = 0; j < pq_dim; j++) {
      for (uint32_t b = 0; b < bits; b++) {
        if ((codes[i * pq_dim + j] >> b) & 1u) {
          const size_t bit = size_t(j) * bits + b;
          out[i * row_bytes + bit / 8] |= uint8_t(1u << (bit % 8));
        }
      }
    }
  }
  return out;
}

struct search_result {
  std::vector<int64_t> ids;
  std::vector<float> dist;
};

search_result search_all(cuvs::resources& res, const ivf_pq::index<int64_t>& index, const float* d_queries,
                         int64_t n_queries, int64_t k)
{
  ivf_pq::search_params sp;
  sp.n_probes  = index.n_lists();
  auto* d_ids  = device_array<int64_t>(n_queries * k);
  auto* d_dist = device_array<float>(n_queries * k);
  ivf_pq::search<float>(res, sp, index, make_device_matrix_view<const float>(d_queries, n_queries, index.dim()),
                        make_device_matrix_view(d_ids, n_queries, k), make_device_matrix_view(d_dist, n_queries, k));
  res.sync();
  search_result r{to_host(d_ids, n_queries * k), to_host(d_dist, n_queries * k)};
  REQUIRE(hipFree(d_ids) == hipSuccess && hipFree(d_dist) == hipSuccess);
  return r;
}

template <typename Fn>
bool throws(Fn fn)
{
  try {
    fn();
  } catch (const cuvs::logic_error&) {
    return true;
  }
  return false;
}

void run(uint32_t pq_bits, ivf_pq::codebook_gen kind, uint32_t pq_dim_asked, const std::vector<float>& data,
         int64_t n_rows, uint32_t dim)
{
  std::printf("pq_bits %u, pq_dim %u, %s codebooks\n", pq_bits, pq_dim_asked,
              kind == ivf_pq::codebook_gen::PER_SUBSPACE ? "per-subspace" : "per-cluster");
  std::fflush(stdout);
  cuvs::resources res;
  float* d_data = to_device(data);
  ivf_pq::index_params ip;
  ip.n_lists       = 40;
  ip.pq_dim        = pq_dim_asked;
  ip.pq_bits       = pq_bits;
  ip.codebook_kind = kind;
  auto index       = ivf_pq::build<float>(res, ip, make_device_matrix_view<const float>(d_data, n_rows, dim));
  REQUIRE(index.size() == n_rows);
  const uint32_t pq_dim = index.pq_dim(), pq_len = index.pq_len(), rot_dim = index.rot_dim();
  const uint32_t book = index.pq_book_size(), n_lists = index.n_lists();
  const size_t row_bytes = (pq_dim * pq_bits + 7) / 8;

  // the largest list
  auto sizes     = to_host(index.list_sizes(), n_lists);
  uint32_t label = uint32_t(std::max_element(sizes.begin(), sizes.end()) - sizes.begin());
  const uint32_t n = sizes[label];
  REQUIRE(n >= 64);
  const int64_t n_queries = 200, k = 10;
  const auto before_search = search_all(res, index, d_data, n_queries, k);
  const auto before        = snapshot(index, label);

  /* unpacking: one code per byte, by range and by position, and bit-contiguous rows */
  auto* d_codes = device_array<uint8_t>(size_t(n) * pq_dim);
  packer::unpack_list_data(res, index, make_device_matrix_view(d_codes, n, pq_dim), label, 0);
  res.sync();
  const auto codes = to_host(d_codes, size_t(n) * pq_dim);
  for (uint8_t c : codes) { REQUIRE(c < book); }
  auto* d_part = device_array<uint8_t>(size_t(20) * pq_dim);
  packer::unpack_list_data(res, index, make_device_matrix_view(d_part, 20, pq_dim), label, 37);
  res.sync();
  REQUIRE(to_host(d_part, size_t(20) * pq_dim) ==
          std::vector<uint8_t>(codes.begin() + 37 * pq_dim, codes.begin() + 57 * pq_dim));
  {
    // the same through the bare-buffer calls: reading the index's own list buffer, and a round trip
    // through a scratch buffer of four groups of 32 rows
    auto ptrs = to_host(index.data_ptrs(), n_lists);
    packer::unpack(res, ptrs[label], pq_bits, 37, make_device_matrix_view(d_part, 20, pq_dim));
    res.sync();
    REQUIRE(to_host(d_part, size_t(20) * pq_dim) ==
            std::vector<uint8_t>(codes.begin() + 37 * pq_dim, codes.begin() + 57 * pq_dim));
    const uint32_t cpc = 128 / pq_bits, n_chunks = (pq_dim + cpc - 1) / cpc;
    auto* d_buf = device_array<uint8_t>(size_t(4) * n_chunks * 512);
    REQUIRE(hipMemset(d_buf, 0, size_t(4) * n_chunks * 512) == hipSuccess);
    packer::pack(res, make_device_matrix_view<const uint8_t>(d_codes, 60, pq_dim), pq_bits, 50, d_buf);
    auto* d_back = device_array<uint8_t>(size_t(60) * pq_dim);
    packer::unpack(res, d_buf, pq_bits, 50, make_device_matrix_view(d_back, 60, pq_dim));
    res.sync();
    REQUIRE(to_host(d_back, size_t(60) * pq_dim) == std::vector<uint8_t>(codes.begin(), codes.begin() + 60 * pq_dim));
    REQUIRE(throws([&] { packer::unpack(res, d_buf, 9, 0, make_device_matrix_view(d_back, 4, pq_dim)); }));
    REQUIRE(hipFree(d_buf) == hipSuccess && hipFree(d_back) == hipSuccess);
  }
  const std::vector<uint32_t> picks = {3, 0, n - 1, 33, 32, 3};
  uint32_t* d_picks = to_device(picks);
  packer::unpack_list_data(res, index, make_device_vector_view<const uint32_t>(d_picks, picks.size()),
                           make_device_matrix_view(d_part, picks.size(), pq_dim), label);
  res.sync();
  const auto picked = to_host(d_part, picks.size() * pq_dim);
  for (size_t i = 0; i < picks.size(); i++) {
    REQUIRE(std::equal(picked.begin() + i * pq_dim, picked.begin() + (i + 1) * pq_dim, codes.begin() + size_t(picks[i]) * pq_dim));
  }
  auto* d_flat = device_array<uint8_t>(size_t(n) * row_bytes);
  packer::unpack_contiguous_list_data(res, index, d_flat, n, label, 0);
  res.sync();
  const auto flat = to_host(d_flat, size_t(n) * row_bytes);
  REQUIRE(flat == contiguous_rows(codes, n, pq_dim, pq_bits));
  {
    // bit strings through the bare-buffer calls: the index's own list buffer read from row 37 on,
    // and rows 5 .. 64 of a scratch buffer written and read back
    auto ptrs = to_host(index.data_ptrs(), n_lists);
    auto* d_rows = device_array<uint8_t>(size_t(60) * row_bytes);
    packer::unpack_contiguous(res, ptrs[label], pq_bits, 37, 20, pq_dim, d_rows);
    res.sync();
    REQUIRE(to_host(d_rows, size_t(20) * row_bytes) ==
            std::vector<uint8_t>(flat.begin() + 37 * row_bytes, flat.begin() + 57 * row_bytes));
    const uint32_t cpc = 128 / pq_bits, n_chunks = (pq_dim + cpc - 1) / cpc;
    auto* d_buf = device_array<uint8_t>(size_t(3) * n_chunks * 512);
    REQUIRE(hipMemset(d_buf, 0, size_t(3) * n_chunks * 512) == hipSuccess);
    packer::pack_contiguous(res, d_flat, 60, pq_dim, pq_bits, 5, d_buf);
    packer::unpack_contiguous(res, d_buf, pq_bits, 5, 60, pq_dim, d_rows);
    res.sync();
    REQUIRE(to_host(d_rows, size_t(60) * row_bytes) == std::vector<uint8_t>(flat.begin(), flat.begin() + 60 * row_bytes));
    // and the byte-per-code reading of the same buffer agrees
    auto* d_back = device_array<uint8_t>(size_t(60) * pq_dim);
    packer::unpack(res, d_buf, pq_bits, 5, make_device_matrix_view(d_back, 60, pq_dim));
    res.sync();
    REQUIRE(to_host(d_back, size_t(60) * pq_dim) == std::vector<uint8_t>(codes.begin(), codes.begin() + 60 * pq_dim));
    REQUIRE(throws([&] { packer::pack_contiguous(res, d_flat, 4, pq_dim, 3, 0, d_buf); }));
    REQUIRE(hipFree(d_buf) == hipSuccess && hipFree(d_back) == hipSuccess && hipFree(d_rows) == hipSuccess);
  }

  /* check_packing: erase the list, put the rows back from their codes: the same bytes */
  int64_t* d_ids = to_device(before.ids);
  ivf_pq::helpers::erase_list(res, &index, label);
  REQUIRE(index.size() == n_rows - int64_t(n));
  REQUIRE(to_host(index.list_sizes(), n_lists)[label] == 0);
  packer::extend_list_with_codes(res, &index, make_device_matrix_view<const uint8_t>(d_codes, n, pq_dim),
                                 make_device_vector_view<const int64_t>(d_ids, n), label);
  REQUIRE(index.size() == n_rows);
  auto after = snapshot(index, label);
  REQUIRE(after.size == n && after.ids == before.ids && after.bytes == before.bytes);
  // the other lists came through the moves unchanged: every query finds what it found
  auto again = search_all(res, index, d_data, n_queries, k);
  REQUIRE(again.ids == before_search.ids && again.dist == before_search.dist);
  // a few rows written again in place
  packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes + 5 * pq_dim, 3, pq_dim), label, 5);
  packer::pack_contiguous_list_data(res, &index, d_flat + 40 * row_bytes, 9, label, 40);
  REQUIRE(snapshot(index, label).bytes == before.bytes);
  {
    // The same kind of edit through a bare pointer into the index's own list buffer: searches read
    // copies of the lists' leading codes (and of 5 - 7-bit codes a byte each), which have to follow.
    // (every row of the list takes the codes of the row after it: the queries that are rows of this
    // list find other neighbours then)
    auto ptrs       = to_host(index.data_ptrs(), n_lists);
    uint8_t* own    = const_cast<uint8_t*>(ptrs[label]);
    packer::pack(res, make_device_matrix_view<const uint8_t>(d_codes + pq_dim, n - 1, pq_dim), pq_bits, 0, own);
    packer::pack(res, make_device_matrix_view<const uint8_t>(d_codes, 1, pq_dim), pq_bits, n - 1, own);
    const auto bare = search_all(res, index, d_data, n_queries, k);
    packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes, n, pq_dim), label, 0);
    REQUIRE(snapshot(index, label).bytes == before.bytes);
    packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes + pq_dim, n - 1, pq_dim), label, 0);
    packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes, 1, pq_dim), label, n - 1);
    const auto proper = search_all(res, index, d_data, n_queries, k);
    REQUIRE(bare.ids == proper.ids && bare.dist == proper.dist);
    REQUIRE(!(proper.ids == before_search.ids && proper.dist == before_search.dist));  // the edit is visible at all
    // bit strings the same way, back to the original rows
    packer::pack_contiguous(res, d_flat, n, pq_dim, pq_bits, 0, own);
    const auto restored = search_all(res, index, d_data, n_queries, k);
    REQUIRE(restored.ids == before_search.ids && restored.dist == before_search.dist);
    REQUIRE(snapshot(index, label).bytes == before.bytes);
  }
  // rows written somewhere else do change the list, and exactly those rows
  packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes + 5 * pq_dim, 3, pq_dim), label, 10);
  packer::unpack_list_data(res, index, make_device_matrix_view(d_part, 20, pq_dim), label, 0);
  res.sync();
  auto moved = to_host(d_part, size_t(20) * pq_dim);
  for (uint32_t i = 0; i < 20; i++) {
    const uint32_t src = (i >= 10 && i < 13) ? i - 5 : i;
    REQUIRE(std::equal(moved.begin() + i * pq_dim, moved.begin() + (i + 1) * pq_dim, codes.begin() + size_t(src) * pq_dim));
  }
  packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes + 10 * pq_dim, 3, pq_dim), label, 10);
  REQUIRE(snapshot(index, label).bytes == before.bytes);
  // the list resized by hand: 40 more rows (empty slots until written), then the old size again
  ivf_pq::helpers::resize_list(res, &index, label, n + 40);
  REQUIRE(index.size() == n_rows + 40 && to_host(index.list_sizes(), n_lists)[label] == n + 40);
  {
    const auto grown = snapshot(index, label);
    REQUIRE(std::equal(before.ids.begin(), before.ids.end(), grown.ids.begin()));
    for (uint32_t i = n; i < n + 40; i++) { REQUIRE(grown.ids[i] == -1); }
    packer::unpack_list_data(res, index, make_device_matrix_view(d_codes, n, pq_dim), label, 0);
    res.sync();
    REQUIRE(to_host(d_codes, size_t(n) * pq_dim) == codes);
    // written like any other rows of the list
    packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes, 40, pq_dim), label, n);
    packer::unpack_list_data(res, index, make_device_matrix_view(d_part, 20, pq_dim), label, n + 20);
    res.sync();
    REQUIRE(to_host(d_part, size_t(20) * pq_dim) ==
            std::vector<uint8_t>(codes.begin() + 20 * pq_dim, codes.begin() + 40 * pq_dim));
  }
  ivf_pq::helpers::resize_list(res, &index, label, n);
  REQUIRE(index.size() == n_rows);
  after = snapshot(index, label);
  REQUIRE(after.size == n && after.ids == before.ids && after.bytes == before.bytes);
  again = search_all(res, index, d_data, n_queries, k);
  REQUIRE(again.ids == before_search.ids && again.dist == before_search.dist);
  REQUIRE(throws([&] { ivf_pq::helpers::resize_list(res, &index, n_lists, 1); }));
  // the same from bit-contiguous rows, in two parts: the second fits the padding or moves the lists
  ivf_pq::helpers::erase_list(res, &index, label);
  const uint32_t first_part = n - 7;
  packer::extend_list_with_contiguous_codes(res, &index, make_device_matrix_view<const uint8_t>(d_flat, first_part, row_bytes),
                                            make_device_vector_view<const int64_t>(d_ids, first_part), label);
  packer::extend_list_with_contiguous_codes(
    res, &index, make_device_matrix_view<const uint8_t>(d_flat + size_t(first_part) * row_bytes, 7, row_bytes),
    make_device_vector_view<const int64_t>(d_ids + first_part, 7), label);
  after = snapshot(index, label);
  REQUIRE(after.size == n && after.ids == before.ids && after.bytes == before.bytes);
  again = search_all(res, index, d_data, n_queries, k);
  REQUIRE(again.ids == before_search.ids && again.dist == before_search.dist);

  /* growing a list in place (the padding of its last group) and by moving the arenas */
  {
    auto grow_by = [&](uint32_t extra) {
      const uint32_t size0 = to_host(index.list_sizes(), n_lists)[label];
      packer::extend_list_with_codes(res, &index, make_device_matrix_view<const uint8_t>(d_codes, extra, pq_dim),
                                     make_device_vector_view<const int64_t>(d_ids, extra), label);
      const auto now = snapshot(index, label);
      REQUIRE(now.size == size0 + extra && index.size() == n_rows + int64_t(size0 + extra - n));
      REQUIRE(std::equal(now.ids.begin(), now.ids.begin() + n, before.ids.begin()));
      REQUIRE(std::equal(now.ids.begin() + size0, now.ids.end(), before.ids.begin()));
      auto* d_tail = device_array<uint8_t>(size_t(extra) * pq_dim);
      packer::unpack_list_data(res, index, make_device_matrix_view(d_tail, extra, pq_dim), label, size0);
      res.sync();
      REQUIRE(to_host(d_tail, size_t(extra) * pq_dim) == std::vector<uint8_t>(codes.begin(), codes.begin() + size_t(extra) * pq_dim));
      packer::unpack_list_data(res, index, make_device_matrix_view(d_part, 20, pq_dim), label, 37);
      res.sync();
      REQUIRE(to_host(d_part, size_t(20) * pq_dim) == std::vector<uint8_t>(codes.begin() + 37 * pq_dim, codes.begin() + 57 * pq_dim));
      REQUIRE(hipFree(d_tail) == hipSuccess);
    };
    grow_by(1);
    grow_by(40);
    grow_by(31);
    grow_by(32 - (n + 72) % 32);  // up to a group boundary exactly
    grow_by(1);
    ivf_pq::helpers::erase_list(res, &index, label);
    packer::extend_list_with_codes(res, &index, make_device_matrix_view<const uint8_t>(d_codes, n, pq_dim),
                                   make_device_vector_view<const int64_t>(d_ids, n), label);
    after = snapshot(index, label);
    REQUIRE(after.size == n && after.ids == before.ids && after.bytes == before.bytes);
    again = search_all(res, index, d_data, n_queries, k);
    REQUIRE(again.ids == before_search.ids && again.dist == before_search.dist);
  }

  /* check_reconstruction: decoded rows against the closed form, and near the rows they encode */
  const auto rotation    = to_host(index.rotation_matrix(), size_t(rot_dim) * dim);
  const auto centers_rot = to_host(index.centers_rot(), size_t(n_lists) * rot_dim);
  const size_t n_books   = kind == ivf_pq::codebook_gen::PER_SUBSPACE ? pq_dim : n_lists;
  const auto books       = to_host(index.pq_centers(), n_books * pq_len * book);
  const uint32_t n_take = 50, n_skip = 3;
  std::vector<double> want(size_t(n_take) * dim, 0.0);
  for (uint32_t i = 0; i < n_take; i++) {
    for (uint32_t j = 0; j < pq_dim; j++) {
      const size_t part = kind == ivf_pq::codebook_gen::PER_SUBSPACE ? j : label;
      for (uint32_t t = 0; t < pq_len; t++) {
        const uint32_t r = j * pq_len + t;
        const double y   = double(centers_rot[size_t(label) * rot_dim + r]) +
                         double(books[(part * pq_len + t) * book + codes[size_t(n_skip + i) * pq_dim + j]]);
        for (uint32_t d = 0; d < dim; d++) { want[size_t(i) * dim + d] += double(rotation[size_t(r) * dim + d]) * y; }
      }
    }
  }
  auto* d_rec = device_array<float>(size_t(n) * dim);
  packer::reconstruct_list_data<float>(res, index, make_device_matrix_view(d_rec, n_take, dim), label, n_skip);
  const auto rec = to_host(d_rec, size_t(n_take) * dim);
  double err2 = 0.0, spread2 = 0.0;
  std::vector<float> centre(dim);
  {
    const auto ext = to_host(index.centers(), size_t(n_lists) * index.dim_ext());
    std::copy(ext.begin() + size_t(label) * index.dim_ext(), ext.begin() + size_t(label) * index.dim_ext() + dim, centre.begin());
  }
  for (uint32_t i = 0; i < n_take; i++) {
    const float* orig = data.data() + size_t(before.ids[n_skip + i]) * dim;
    for (uint32_t d = 0; d < dim; d++) {
      REQUIRE(std::fabs(double(rec[size_t(i) * dim + d]) - want[size_t(i) * dim + d]) <= 1e-4 * (1.0 + std::fabs(want[size_t(i) * dim + d])));
      err2 += std::pow(double(rec[size_t(i) * dim + d]) - double(orig[d]), 2);
      spread2 += std::pow(double(orig[d]) - double(centre[d]), 2);
    }
  }
  REQUIRE(err2 < (pq_bits == 8 ? 0.5 : 0.9) * spread2);  // the codes say more about a row than its list alone
  // by position
  packer::reconstruct_list_data<float>(res, index, make_device_vector_view<const uint32_t>(d_picks, picks.size()),
                                       make_device_matrix_view(d_rec, picks.size(), dim), label);
  const auto rec_picked = to_host(d_rec, picks.size() * dim);
  for (size_t i = 0; i < picks.size(); i++) {
    if (picks[i] >= n_skip && picks[i] < n_skip + n_take) {
      REQUIRE(std::equal(rec_picked.begin() + i * dim, rec_picked.begin() + (i + 1) * dim, rec.begin() + size_t(picks[i] - n_skip) * dim));
    }
  }
  REQUIRE(std::equal(rec_picked.begin(), rec_picked.begin() + dim, rec_picked.begin() + 5 * dim));  // position 3 twice
  // integer element types: the float result scaled back and clamped (binary16 output needs a
  // compiler with _Float16 on the caller's side and is left out of this program)
  auto* d_i8   = device_array<int8_t>(size_t(n_take) * dim);
  auto* d_u8   = device_array<uint8_t>(size_t(n_take) * dim);
  packer::reconstruct_list_data<int8_t>(res, index, make_device_matrix_view(d_i8, n_take, dim), label, n_skip);
  packer::reconstruct_list_data<uint8_t>(res, index, make_device_matrix_view(d_u8, n_take, dim), label, n_skip);
  const auto i8   = to_host(d_i8, size_t(n_take) * dim);
  const auto u8   = to_host(d_u8, size_t(n_take) * dim);
  for (size_t e = 0; e < size_t(n_take) * dim; e++) {
    REQUIRE(i8[e] == static_cast<int8_t>(std::min(std::max(rec[e] * 128.0f, -128.0f), 127.0f)));
    REQUIRE(u8[e] == static_cast<uint8_t>(std::min(std::max(rec[e] * 256.0f, 0.0f), 255.0f)));
  }

  /* check_reconstruct_extend: decode the list, erase it, encode the decoded rows into it */
  packer::reconstruct_list_data<float>(res, index, make_device_matrix_view(d_rec, n, dim), label, 0);
  const auto vectors_1 = to_host(d_rec, size_t(n) * dim);
  ivf_pq::helpers::erase_list(res, &index, label);
  packer::extend_list<float>(res, &index, make_device_matrix_view<const float>(d_rec, n, dim),
                             make_device_vector_view<const int64_t>(d_ids, n), label);
  after = snapshot(index, label);
  REQUIRE(after.size == n && after.ids == before.ids);  // in the order given
  auto* d_codes_2 = device_array<uint8_t>(size_t(n) * pq_dim);
  packer::unpack_list_data(res, index, make_device_matrix_view(d_codes_2, n, pq_dim), label, 0);
  auto* d_rec_2 = device_array<float>(size_t(n) * dim);
  packer::reconstruct_list_data<float>(res, index, make_device_matrix_view(d_rec_2, n, dim), label, 0);
  const auto codes_2   = to_host(d_codes_2, size_t(n) * pq_dim);
  const auto vectors_2 = to_host(d_rec_2, size_t(n) * dim);
  size_t same_codes = 0;
  for (size_t e = 0; e < codes.size(); e++) { same_codes += codes[e] == codes_2[e]; }
  // a decoded row is a codebook entry away from nothing: it encodes to itself unless entries coincide
  REQUIRE(same_codes >= codes.size() * 99 / 100);
  double diff2 = 0.0, norm2 = 0.0;
  for (size_t e = 0; e < vectors_1.size(); e++) {
    diff2 += std::pow(double(vectors_1[e]) - double(vectors_2[e]), 2);
    norm2 += std::pow(double(vectors_1[e]), 2);
  }
  REQUIRE(diff2 <= 1e-3 * norm2);

  /* centres, errors, reset */
  std::vector<float> centres(size_t(n_lists) * dim);
  ivf_pq::helpers::extract_centers(res, index, centres.data());
  res.sync();
  const auto ext = to_host(index.centers(), size_t(n_lists) * index.dim_ext());
  for (uint32_t l = 0; l < n_lists; l++) {
    REQUIRE(std::equal(centres.begin() + size_t(l) * dim, centres.begin() + size_t(l + 1) * dim, ext.begin() + size_t(l) * index.dim_ext()));
  }
  REQUIRE(throws([&] { packer::unpack_list_data(res, index, make_device_matrix_view(d_codes, n, pq_dim), n_lists, 0); }));
  REQUIRE(throws([&] { packer::unpack_list_data(res, index, make_device_matrix_view(d_codes, n, pq_dim), label, 1); }));
  REQUIRE(throws([&] { packer::unpack_list_data(res, index, make_device_matrix_view(d_codes, 2, pq_dim + 1), label, 0); }));
  REQUIRE(throws([&] { packer::pack_list_data(res, &index, make_device_matrix_view<const uint8_t>(d_codes, 3, pq_dim), label, n - 2); }));
  REQUIRE(throws([&] { packer::reconstruct_list_data<float>(res, index, make_device_matrix_view(d_rec, 4, dim + 1), label, 0); }));
  REQUIRE(throws([&] { ivf_pq::helpers::erase_list(res, &index, n_lists); }));
  ivf_pq::helpers::reset_index(res, &index);
  REQUIRE(index.size() == 0);
  for (uint32_t s : to_host(index.list_sizes(), n_lists)) { REQUIRE(s == 0); }
  REQUIRE(throws([&] { search_all(res, index, d_data, 5, k); }));  // k exceeds the size of the index
  ivf_pq::extend<float>(res, make_device_matrix_view<const float>(d_data, n_rows, dim), nullptr, &index);
  ivf_pq::helpers::recompute_internal_state(res, &index);
  REQUIRE(index.size() == n_rows);
  again = search_all(res, index, d_data, n_queries, k);
  REQUIRE(again.dist == before_search.dist);  // the same rows under the same model

  /* copies: a clone is independent of its source; extend that returns an index leaves `orig` alone */
  {
    const auto base = search_all(res, index, d_data, n_queries, k);
    auto copy       = ivf_pq::clone(res, index);
    const auto same = search_all(res, copy, d_data, n_queries, k);
    REQUIRE(same.ids == base.ids && same.dist == base.dist);
    ivf_pq::helpers::erase_list(res, &copy, label);
    REQUIRE(copy.size() == n_rows - int64_t(to_host(index.list_sizes(), n_lists)[label]) && index.size() == n_rows);
    auto grown = ivf_pq::extend<float>(res, make_device_matrix_view<const float>(d_data, 500, dim), nullptr, index);
    REQUIRE(index.size() == n_rows && grown.size() == n_rows + 500);
    const auto still = search_all(res, index, d_data, n_queries, k);
    REQUIRE(still.ids == base.ids && still.dist == base.dist);
    // rows 0 .. 499 are in `grown` twice, as ids i and n_rows + i, with the same code in the same list
    const auto twice = search_all(res, grown, d_data, n_queries, k);
    for (int64_t q = 0; q < n_queries; q++) {
      for (int64_t r = 0; r + 1 < k; r++) {
        const int64_t id = twice.ids[q * k + r];
        if (id >= 500 && id < n_rows) { continue; }
        const int64_t twin = id < 500 ? id + n_rows : id - n_rows;
        REQUIRE(std::count(twice.ids.begin() + q * k, twice.ids.begin() + (q + 1) * k, twin) == 1 ||
                twice.dist[q * k + r] == twice.dist[q * k + k - 1]);
      }
    }
    ivf_pq::index<int64_t> held;
    ivf_pq::index_params untrained = ip;
    untrained.add_data_on_build    = false;
    ivf_pq::build<float>(res, untrained, make_device_matrix_view<const float>(d_data, n_rows, dim), &held);
    REQUIRE(held.n_lists() == n_lists && held.size() == 0 && held.pq_bits() == pq_bits);
  }

  /* a model put together from its parts with the centre / rotation helpers is the trained model */
  {
    const uint32_t dim_ext = index.dim_ext();
    auto* d_flat_centres   = device_array<float>(size_t(n_lists) * dim);
    ivf_pq::helpers::extract_centers(res, index, d_flat_centres);
    auto* d_padded  = device_array<float>(size_t(n_lists) * dim_ext);
    auto* d_padded2 = device_array<float>(size_t(n_lists) * dim_ext);
    ivf_pq::helpers::pad_centers_with_norms(res, make_device_matrix_view<const float>(d_flat_centres, n_lists, dim),
                                            make_device_matrix_view(d_padded, n_lists, dim_ext));
    ivf_pq::helpers::pad_centers_with_norms(res, make_device_matrix_view<const float>(centres.data(), n_lists, dim),
                                            make_device_matrix_view(d_padded2, n_lists, dim_ext));  // from the host
    const auto padded = to_host(d_padded, size_t(n_lists) * dim_ext);
    REQUIRE(padded == to_host(d_padded2, size_t(n_lists) * dim_ext));
    for (uint32_t l = 0; l < n_lists; l++) {
      double ss = 0.0;
      for (uint32_t d = 0; d < dim; d++) {
        REQUIRE(padded[size_t(l) * dim_ext + d] == centres[size_t(l) * dim + d]);
        ss += double(centres[size_t(l) * dim + d]) * double(centres[size_t(l) * dim + d]);
      }
      REQUIRE(std::fabs(double(padded[size_t(l) * dim_ext + dim]) - ss) <= 1e-5 * ss);
      for (uint32_t d = dim + 1; d < dim_ext; d++) { REQUIRE(padded[size_t(l) * dim_ext + d] == 0.0f); }
    }
    auto* d_rotation = device_array<float>(size_t(rot_dim) * dim);
    ivf_pq::helpers::make_rotation_matrix(res, make_device_matrix_view(d_rotation, rot_dim, dim), false);
    REQUIRE(to_host(d_rotation, size_t(rot_dim) * dim) == rotation);  // rot_dim == dim here: the identity
    auto* d_rotated = device_array<float>(size_t(n_lists) * rot_dim);
    ivf_pq::helpers::rotate_padded_centers(res, make_device_matrix_view<const float>(d_padded, n_lists, dim_ext),
                                           make_device_matrix_view<const float>(d_rotation, rot_dim, dim),
                                           make_device_matrix_view(d_rotated, n_lists, rot_dim));
    REQUIRE(to_host(d_rotated, size_t(n_lists) * rot_dim) == centers_rot);
    auto rebuilt = ivf_pq::build(res, ip, dim, index.pq_centers(), d_padded, d_rotated, d_rotation);
    ivf_pq::extend<float>(res, make_device_matrix_view<const float>(d_data, n_rows, dim), nullptr, &rebuilt);
    const auto base = search_all(res, index, d_data, n_queries, k);
    const auto same = search_all(res, rebuilt, d_data, n_queries, k);
    REQUIRE(same.dist == base.dist);
    // a random rotation to a wider space: orthonormal columns, and rotated centres = R c
    const uint32_t wide = dim + 8;
    auto* d_wide = device_array<float>(size_t(wide) * dim);
    ivf_pq::helpers::make_rotation_matrix(res, make_device_matrix_view(d_wide, wide, dim), true);
    const auto r = to_host(d_wide, size_t(wide) * dim);
    for (uint32_t a = 0; a < dim; a++) {
      for (uint32_t b = 0; b <= a; b++) {
        double dot = 0.0;
        for (uint32_t o = 0; o < wide; o++) { dot += double(r[size_t(o) * dim + a]) * double(r[size_t(o) * dim + b]); }
        REQUIRE(std::fabs(dot - (a == b ? 1.0 : 0.0)) < 1e-5);
      }
    }
    auto* d_rotated_wide = device_array<float>(size_t(n_lists) * wide);
    ivf_pq::helpers::rotate_padded_centers(res, make_device_matrix_view<const float>(d_padded, n_lists, dim_ext),
                                           make_device_matrix_view<const float>(d_wide, wide, dim),
                                           make_device_matrix_view(d_rotated_wide, n_lists, wide));
    const auto rotated_wide = to_host(d_rotated_wide, size_t(n_lists) * wide);
    for (uint32_t l = 0; l < n_lists; l += 7) {
      for (uint32_t o = 0; o < wide; o++) {
        double y = 0.0;
        for (uint32_t d = 0; d < dim; d++) { y += double(r[size_t(o) * dim + d]) * double(centres[size_t(l) * dim + d]); }
        REQUIRE(std::fabs(double(rotated_wide[size_t(l) * wide + o]) - y) < 1e-5);
      }
    }
    for (void* p : {static_cast<void*>(d_flat_centres), static_cast<void*>(d_padded), static_cast<void*>(d_padded2),
                    static_cast<void*>(d_rotation), static_cast<void*>(d_rotated), static_cast<void*>(d_wide),
                    static_cast<void*>(d_rotated_wide)}) {
      REQUIRE(hipFree(p) == hipSuccess);
    }
  }

  for (void* p : {static_cast<void*>(d_data), static_cast<void*>(d_codes), static_cast<void*>(d_part), static_cast<void*>(d_picks),
                  static_cast<void*>(d_flat), static_cast<void*>(d_ids), static_cast<void*>(d_rec),
                  static_cast<void*>(d_i8), static_cast<void*>(d_u8), static_cast<void*>(d_codes_2), static_cast<void*>(d_rec_2)}) {
    REQUIRE(hipFree(p) == hipSuccess);
  }
}

}  // namespace

int main()
{
  constexpr int64_t n_rows = 20000;
  constexpr uint32_t dim   = 32;
  std::mt19937 gen(11);
  std::normal_distribution<float> noise(0.0f, 0.05f);
  std::uniform_real_distribution<float> place(0.1f, 0.9f);
  std::vector<float> centres(30 * dim), data(n_rows * dim);
  for (auto& v : centres) { v = place(gen); }
  for (int64_t i = 0; i < n_rows; i++) {
    const int c = int(gen() % 30);
    for (uint32_t d = 0; d < dim; d++) { data[i * dim + d] = centres[c * dim + d] + noise(gen); }
  }
  for (uint32_t bits : {8u, 5u, 4u}) {
    run(bits, ivf_pq::codebook_gen::PER_SUBSPACE, 16, data, n_rows, dim);
    run(bits, ivf_pq::codebook_gen::PER_CLUSTER, 16, data, n_rows, dim);
  }
  // rows of more than one 16-byte chunk, the last one partly filled (16, 25, 21 and 18 codes per chunk)
  run(8, ivf_pq::codebook_gen::PER_SUBSPACE, 32, data, n_rows, dim);
  run(5, ivf_pq::codebook_gen::PER_CLUSTER, 32, data, n_rows, dim);
  run(6, ivf_pq::codebook_gen::PER_SUBSPACE, 32, data, n_rows, dim);
  run(7, ivf_pq::codebook_gen::PER_CLUSTER, 32, data, n_rows, dim);
  std::printf("ok\n");
  return 0;
}
