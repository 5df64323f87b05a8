/*
 * A C++17 caller of the C++ interface (cuvs::neighbors::ivf_pq::build / search, refine,
 * knn_merge_parts) compiled by the host compiler alone and linked against the shared library:
 * the flow of the reference's C++ example (build, search, refine the candidates), plus a search
 * over two half-indexes merged into one answer.  Exits 0 when everything agrees.
 *
 *   g++ -std=c++17 -D__HIP_PLATFORM_AMD__ -Iinclude -isystem /opt/rocm/include \
 *       tests/c_abi/ivf_pq_cpp_caller.cpp -Lcuvs_amd -lcuvs_c -L/opt/rocm/lib -lamdhip64 \
 *       -Wl,-rpath,$PWD/cuvs_amd -o /tmp/ivf_pq_cpp_caller
 */
#include <cuvs/neighbors/ivf_pq.hpp>
#include <cuvs/neighbors/knn_merge_parts.hpp>
#include <cuvs/neighbors/refine.hpp>

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <random>
#include <sstream>
#include <vector>

namespace {

template <typename T>
T* to_device(const std::vector<T>& host)
{
  void* ptr = nullptr;
  if (hipMalloc(&ptr, host.size() * sizeof(T)) != hipSuccess) { std::abort(); }
  if (hipMemcpy(ptr, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) { std::abort(); }
  return static_cast<T*>(ptr);
}

template <typename T>
std::vector<T> to_host(const T* device, size_t n)
{
  std::vector<T> host(n);
  if (hipMemcpy(host.data(), device, n * sizeof(T), hipMemcpyDeviceToHost) != hipSuccess) { std::abort(); }
  return host;
}

template <typename T>
T* device_array(size_t n)
{
  void* ptr = nullptr;
  if (hipMalloc(&ptr, n * sizeof(T)) != hipSuccess) { std::abort(); }
  return static_cast<T*>(ptr);
}

}  // namespace

int main()
{
  using namespace cuvs::neighbors;
  constexpr int64_t n_rows = 30000, dim = 64, n_queries = 500, k = 10, k_wide = 40;
  std::mt19937 gen(7);
  std::normal_distribution<float> noise(0.0f, 0.3f);
  std::vector<float> centres(50 * dim), data(n_rows * dim);
  for (auto& v : centres) { v = noise(gen) * 10.0f; }
  for (int64_t i = 0; i < n_rows; i++) {
    const int c = int(gen() % 50);
    for (int64_t d = 0; d < dim; d++) { data[i * dim + d] = centres[c * dim + d] + noise(gen); }
  }
  float* d_data = to_device(data);

  cuvs::resources res;
  ivf_pq::index_params ip;
  ip.n_lists = 100;
  ip.pq_dim  = 32;
  auto index = ivf_pq::build<float>(res, ip, cuvs::make_device_matrix_view<const float>(d_data, n_rows, dim));
  if (index.size() != n_rows || index.n_lists() != 100 || index.pq_dim() != 32) { return 1; }

  // the first rows as queries
  ivf_pq::search_params sp;
  sp.n_probes      = 20;
  auto* d_nb       = device_array<int64_t>(n_queries * k_wide);
  auto* d_dist     = device_array<float>(n_queries * k_wide);
  const auto q_view = cuvs::make_device_matrix_view<const float>(d_data, n_queries, dim);
  ivf_pq::search<float>(res, sp, index, q_view, cuvs::make_device_matrix_view(d_nb, n_queries, k_wide),
                        cuvs::make_device_matrix_view(d_dist, n_queries, k_wide));
  // exact re-ranking of the 40 candidates
  auto* d_ref_nb   = device_array<int64_t>(n_queries * k);
  auto* d_ref_dist = device_array<float>(n_queries * k);
  refine<float>(res, cuvs::make_device_matrix_view<const float>(d_data, n_rows, dim), q_view,
                cuvs::make_device_matrix_view<const int64_t>(d_nb, n_queries, k_wide),
                cuvs::make_device_matrix_view(d_ref_nb, n_queries, k),
                cuvs::make_device_matrix_view(d_ref_dist, n_queries, k));
  res.sync();
  const auto nb   = to_host(d_ref_nb, n_queries * k);
  const auto dist = to_host(d_ref_dist, n_queries * k);
  int self = 0;
  for (int64_t q = 0; q < n_queries; q++) {
    self += nb[q * k] == q && dist[q * k] == 0.0f;
    for (int64_t r = 1; r < k; r++) {
      if (dist[q * k + r] < dist[q * k + r - 1]) { std::fprintf(stderr, "refined distances not ascending\n"); return 1; }
    }
  }
  if (self < n_queries * 95 / 100) { std::fprintf(stderr, "%d of %ld rows found themselves\n", self, long(n_queries)); return 1; }

  // the overload for matrices in host memory: same rows, same distances
  {
    const auto cand = to_host(d_nb, n_queries * k_wide);
    std::vector<int64_t> h_nb(n_queries * k);
    std::vector<float> h_dist(n_queries * k);
    refine<float>(res, cuvs::make_host_matrix_view<const float>(data.data(), n_rows, dim),
                  cuvs::make_host_matrix_view<const float>(data.data(), n_queries, dim),
                  cuvs::make_host_matrix_view<const int64_t>(cand.data(), n_queries, k_wide),
                  cuvs::make_host_matrix_view(h_nb.data(), n_queries, k),
                  cuvs::make_host_matrix_view(h_dist.data(), n_queries, k));
    if (h_nb != nb || h_dist != dist) { std::fprintf(stderr, "host refine differs from device refine\n"); return 1; }
    // and the overloads with 32-bit ids, on the device and in host memory
    std::vector<uint32_t> cand32(cand.begin(), cand.end()), h_nb32(n_queries * k);
    refine(res, cuvs::make_host_matrix_view<const float>(data.data(), n_rows, dim),
           cuvs::make_host_matrix_view<const float>(data.data(), n_queries, dim),
           cuvs::make_host_matrix_view<const uint32_t>(cand32.data(), n_queries, k_wide),
           cuvs::make_host_matrix_view(h_nb32.data(), n_queries, k), cuvs::make_host_matrix_view(h_dist.data(), n_queries, k));
    uint32_t* d_cand32 = to_device(cand32);
    auto* d_nb32       = device_array<uint32_t>(n_queries * k);
    refine(res, cuvs::make_device_matrix_view<const float>(d_data, n_rows, dim), q_view,
           cuvs::make_device_matrix_view<const uint32_t>(d_cand32, n_queries, k_wide),
           cuvs::make_device_matrix_view(d_nb32, n_queries, k), cuvs::make_device_matrix_view(d_ref_dist, n_queries, k));
    res.sync();
    const auto nb32 = to_host(d_nb32, n_queries * k);
    for (int64_t i = 0; i < n_queries * k; i++) {
      if (int64_t(nb32[i]) != nb[i] || int64_t(h_nb32[i]) != nb[i]) { std::fprintf(stderr, "32-bit refine differs at %ld\n", long(i)); return 1; }
    }
    if (h_dist != dist || to_host(d_ref_dist, n_queries * k) != dist) { std::fprintf(stderr, "32-bit refine distances differ\n"); return 1; }
  }

  // the same rows as two half-indexes under one model: merged answers = the whole index's answers
  ivf_pq::index_params empty = ip;
  empty.add_data_on_build    = false;
  auto model = ivf_pq::build<float>(res, empty, cuvs::make_device_matrix_view<const float>(d_data, n_rows, dim));
  auto make_part = [&](int64_t first, int64_t count) {
    auto part = ivf_pq::build(res, empty, uint32_t(dim), model.pq_centers(), model.centers(), model.centers_rot(),
                              model.rotation_matrix());
    ivf_pq::extend<float>(res, cuvs::make_device_matrix_view<const float>(d_data + first * dim, count, dim), nullptr, &part);
    return part;
  };
  auto whole = make_part(0, n_rows);
  auto lo    = make_part(0, n_rows / 2);
  auto hi    = make_part(n_rows / 2, n_rows - n_rows / 2);
  sp.n_probes = 100;  // every list: the candidates of the halves are exactly those of the whole
  auto* d_parts_nb   = device_array<int64_t>(2 * n_queries * k);
  auto* d_parts_dist = device_array<float>(2 * n_queries * k);
  auto* d_whole_nb   = device_array<int64_t>(n_queries * k);
  auto* d_whole_dist = device_array<float>(n_queries * k);
  ivf_pq::search<float>(res, sp, lo, q_view, cuvs::make_device_matrix_view(d_parts_nb, n_queries, k),
                        cuvs::make_device_matrix_view(d_parts_dist, n_queries, k));
  ivf_pq::search<float>(res, sp, hi, q_view, cuvs::make_device_matrix_view(d_parts_nb + n_queries * k, n_queries, k),
                        cuvs::make_device_matrix_view(d_parts_dist + n_queries * k, n_queries, k));
  ivf_pq::search<float>(res, sp, whole, q_view, cuvs::make_device_matrix_view(d_whole_nb, n_queries, k),
                        cuvs::make_device_matrix_view(d_whole_dist, n_queries, k));
  auto* d_merged_nb   = device_array<int64_t>(n_queries * k);
  auto* d_merged_dist = device_array<float>(n_queries * k);
  const std::vector<int64_t> offsets = {0, n_rows / 2};
  int64_t* d_offsets                  = to_device(offsets);
  knn_merge_parts<int64_t>(res, cuvs::make_device_matrix_view<const float>(d_parts_dist, 2 * n_queries, k),
                           cuvs::make_device_matrix_view<const int64_t>(d_parts_nb, 2 * n_queries, k),
                           cuvs::make_device_matrix_view(d_merged_dist, n_queries, k),
                           cuvs::make_device_matrix_view(d_merged_nb, n_queries, k), d_offsets, 2);
  res.sync();
  if (to_host(d_merged_dist, n_queries * k) != to_host(d_whole_dist, n_queries * k)) {
    std::fprintf(stderr, "merged distances differ from the whole index's\n");
    return 1;
  }
  const auto merged_nb = to_host(d_merged_nb, n_queries * k);
  const auto whole_nb  = to_host(d_whole_nb, n_queries * k);
  const auto whole_d   = to_host(d_whole_dist, n_queries * k);
  for (int64_t i = 0; i < n_queries * k; i++) {
    // ids may swap only between equal distances
    const bool tie = (i % k > 0 && whole_d[i] == whole_d[i - 1]) || (i % k < k - 1 && whole_d[i] == whole_d[i + 1]);
    if (merged_nb[i] != whole_nb[i] && !tie) { std::fprintf(stderr, "merged ids differ at %ld\n", long(i)); return 1; }
  }

  // the two halves written to one stream and read back from it: each answers as before
  {
    std::stringstream both(std::ios::in | std::ios::out | std::ios::binary);
    ivf_pq::serialize(res, both, lo);
    ivf_pq::serialize(res, both, hi);
    ivf_pq::index<int64_t> lo2, hi2;
    ivf_pq::deserialize(res, both, &lo2);
    ivf_pq::deserialize(res, both, &hi2);
    if (lo2.size() != lo.size() || hi2.size() != hi.size()) { std::fprintf(stderr, "sizes after the stream differ\n"); return 1; }
    auto* d_nb2   = device_array<int64_t>(2 * n_queries * k);
    auto* d_dist2 = device_array<float>(2 * n_queries * k);
    ivf_pq::search<float>(res, sp, lo2, q_view, cuvs::make_device_matrix_view(d_nb2, n_queries, k),
                          cuvs::make_device_matrix_view(d_dist2, n_queries, k));
    ivf_pq::search<float>(res, sp, hi2, q_view, cuvs::make_device_matrix_view(d_nb2 + n_queries * k, n_queries, k),
                          cuvs::make_device_matrix_view(d_dist2 + n_queries * k, n_queries, k));
    res.sync();
    if (to_host(d_nb2, 2 * n_queries * k) != to_host(d_parts_nb, 2 * n_queries * k) ||
        to_host(d_dist2, 2 * n_queries * k) != to_host(d_parts_dist, 2 * n_queries * k)) {
      std::fprintf(stderr, "indexes read back from a stream answer differently\n");
      return 1;
    }
  }

  // an invalid call throws cuvs::logic_error with a message
  bool thrown = false;
  try {
    sp.n_probes = 0;
    ivf_pq::search<float>(res, sp, whole, q_view, cuvs::make_device_matrix_view(d_whole_nb, n_queries, k),
                          cuvs::make_device_matrix_view(d_whole_dist, n_queries, k));
  } catch (const cuvs::logic_error& e) {
    thrown = std::string(e.what()).find("n_probes") != std::string::npos;
  }
  if (!thrown) { std::fprintf(stderr, "n_probes = 0 was accepted\n"); return 1; }
  std::printf("ok: %d of %ld rows found themselves\n", self, long(n_queries));
  return 0;
}
