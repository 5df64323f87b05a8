/*
 * Index files in the cuVS IVF-PQ format, version 4
 * (cpp/src/neighbors/ivf_pq/ivf_pq_serialize.cuh:41-87 writer, :124-211 reader; per-list records
 * cpp/src/neighbors/ivf_list.cuh:107-176).
 *
 * The file is a sequence of NumPy `.npy` records, one per scalar or array, as written by RAFT's
 * serialize_scalar / serialize_mdspan: magic "\x93NUMPY", version 1.0, a little-endian 16-bit header
 * length, the header dictionary {'descr', 'fortran_order', 'shape'} padded with spaces to a multiple
 * of 64 bytes and ended by '\n', then the raw row-major data.  RAFT's source is not part of the
 * cuVS tree, so the exact padding and the type strings it picks for `bool` and enum scalars are
 * restated from the NumPy format rather than copied: the reader therefore accepts any valid
 * version-1/2 header and checks only element size and element count, and the writer emits headers
 * that NumPy itself reads back.
 *
 * Record order: version (int32), size (int64), dim, pq_bits, pq_dim (uint32), conservative memory
 * allocation (bool), metric, codebook kind, codes layout (int32), n_lists (uint32); pq_centers
 * [pq_dim | n_lists, pq_len, 2^pq_bits], centers [n_lists, dim_ext], centers_rot [n_lists, rot_dim],
 * rotation_matrix [rot_dim, dim] (float32); list_sizes [n_lists] (uint32); then per list its size
 * (uint32) and, when non-empty, its codes [ceil(size / 32), n_chunks, 32, 16] (uint8) and its ids
 * [size] (int64).
 */
#include "detail.hpp"

#include <cstring>
#include <fstream>
#include <string>
#include <vector>

namespace cuvs::neighbors::ivf_pq {

namespace {

constexpr int kSerializationVersion = 4;
const char kMagic[6]                = {'\x93', 'N', 'U', 'M', 'P', 'Y'};

void write_header(std::ostream& os, const char* descr, const std::vector<uint64_t>& shape)
{
  std::string dict = std::string("{'descr': '") + descr + "', 'fortran_order': False, 'shape': (";
  for (size_t i = 0; i < shape.size(); i++) {
    dict += std::to_string(shape[i]);
    if (shape.size() == 1) {
      dict += ",";
    } else if (i + 1 < shape.size()) {
      dict += ", ";
    }
  }
  dict += "), }";
  // magic (6) + version (2) + header length (2) + dictionary + padding + '\n' is a multiple of 64
  const size_t preamble = 6 + 2 + 2 + dict.size() + 1;
  const size_t padding  = (64 - preamble % 64) % 64;
  const uint16_t hlen   = uint16_t(dict.size() + padding + 1);
  os.write(kMagic, 6);
  os.put(char(1));
  os.put(char(0));
  os.put(char(hlen & 0xff));
  os.put(char(hlen >> 8));
  os.write(dict.data(), std::streamsize(dict.size()));
  for (size_t i = 0; i < padding; i++) { os.put(' '); }
  os.put('\n');
}

template <typename T>
void write_scalar(std::ostream& os, const char* descr, T value)
{
  write_header(os, descr, {});
  os.write(reinterpret_cast<const char*>(&value), sizeof(T));
}

void write_array(std::ostream& os, const char* descr, const std::vector<uint64_t>& shape,
                 const void* data, size_t bytes)
{
  write_header(os, descr, shape);
  os.write(static_cast<const char*>(data), std::streamsize(bytes));
}

struct npy_header {
  size_t item_size = 0;
  std::vector<uint64_t> shape;
  uint64_t count() const
  {
    uint64_t n = 1;
    for (auto v : shape) { n *= v; }
    return n;
  }
};

npy_header read_header(std::istream& is, const std::string& what)
{
  char magic[6];
  is.read(magic, 6);
  CUVS_EXPECTS(is.good() && std::memcmp(magic, kMagic, 6) == 0,
               "ivf_pq::deserialize: %s: not a NumPy record (bad magic)", what.c_str());
  const int major = is.get();
  const int minor = is.get();
  CUVS_EXPECTS((major == 1 || major == 2 || major == 3) && minor == 0,
               "ivf_pq::deserialize: %s: unsupported NumPy format version %d.%d", what.c_str(), major,
               minor);
  uint32_t hlen = 0;
  if (major == 1) {
    unsigned char b[2];
    is.read(reinterpret_cast<char*>(b), 2);
    hlen = uint32_t(b[0]) | (uint32_t(b[1]) << 8);
  } else {
    unsigned char b[4];
    is.read(reinterpret_cast<char*>(b), 4);
    hlen = uint32_t(b[0]) | (uint32_t(b[1]) << 8) | (uint32_t(b[2]) << 16) | (uint32_t(b[3]) << 24);
  }
  CUVS_EXPECTS(is.good() && hlen > 0 && hlen < (1u << 20), "ivf_pq::deserialize: %s: bad header length",
               what.c_str());
  std::string dict(hlen, '\0');
  is.read(&dict[0], std::streamsize(hlen));
  CUVS_EXPECTS(is.good(), "ivf_pq::deserialize: %s: truncated header", what.c_str());

  npy_header h;
  // 'descr': '<f4' -> byte order / kind / size
  size_t p = dict.find("'descr'");
  CUVS_EXPECTS(p != std::string::npos, "ivf_pq::deserialize: %s: header without descr", what.c_str());
  p = dict.find('\'', dict.find(':', p));
  const size_t e = dict.find('\'', p + 1);
  CUVS_EXPECTS(p != std::string::npos && e != std::string::npos && e > p + 2,
               "ivf_pq::deserialize: %s: malformed descr", what.c_str());
  const std::string descr = dict.substr(p + 1, e - p - 1);
  CUVS_EXPECTS(descr[0] == '<' || descr[0] == '|' || descr[0] == '=',
               "ivf_pq::deserialize: %s: big-endian data is not supported (%s)", what.c_str(),
               descr.c_str());
  h.item_size = size_t(std::strtoul(descr.c_str() + 2, nullptr, 10));
  CUVS_EXPECTS(h.item_size >= 1 && h.item_size <= 16, "ivf_pq::deserialize: %s: bad element size (%s)",
               what.c_str(), descr.c_str());
  p = dict.find("'fortran_order'");
  CUVS_EXPECTS(p != std::string::npos && dict.compare(dict.find(':', p) + 1, 6, " False") == 0,
               "ivf_pq::deserialize: %s: column-major records are not supported", what.c_str());
  p = dict.find("'shape'");
  CUVS_EXPECTS(p != std::string::npos, "ivf_pq::deserialize: %s: header without shape", what.c_str());
  p              = dict.find('(', p);
  const size_t q = dict.find(')', p);
  CUVS_EXPECTS(p != std::string::npos && q != std::string::npos,
               "ivf_pq::deserialize: %s: malformed shape", what.c_str());
  const char* c = dict.c_str() + p + 1;
  const char* z = dict.c_str() + q;
  while (c < z) {
    while (c < z && (*c == ' ' || *c == ',')) { c++; }
    if (c >= z) { break; }
    char* end = nullptr;
    h.shape.push_back(std::strtoull(c, &end, 10));
    CUVS_EXPECTS(end != c, "ivf_pq::deserialize: %s: malformed shape", what.c_str());
    c = end;
    if (c < z && *c == 'L') { c++; }
  }
  return h;
}

template <typename T>
T read_scalar(std::istream& is, const std::string& what)
{
  const npy_header h = read_header(is, what);
  CUVS_EXPECTS(h.count() == 1 && h.item_size == sizeof(T),
               "ivf_pq::deserialize: %s: expected one %zu-byte value", what.c_str(), sizeof(T));
  T v{};
  is.read(reinterpret_cast<char*>(&v), sizeof(T));
  CUVS_EXPECTS(is.good(), "ivf_pq::deserialize: %s: truncated file", what.c_str());
  return v;
}

void read_array(std::istream& is, const std::string& what, size_t item_size, uint64_t count,
                void* dst)
{
  const npy_header h = read_header(is, what);
  CUVS_EXPECTS(h.item_size == item_size && h.count() == count,
               "ivf_pq::deserialize: %s: expected %llu elements of %zu bytes, found %llu of %zu",
               what.c_str(), static_cast<unsigned long long>(count), item_size,
               static_cast<unsigned long long>(h.count()), h.item_size);
  is.read(static_cast<char*>(dst), std::streamsize(count * item_size));
  CUVS_EXPECTS(is.good(), "ivf_pq::deserialize: %s: truncated file", what.c_str());
}

}  // namespace

void serialize(cuvs::resources const& res, const std::string& filename, const index<int64_t>& idx)
{
  std::ofstream os(filename, std::ios::out | std::ios::binary);
  CUVS_EXPECTS(bool(os), "Cannot open file %s", filename.c_str());
  serialize(res, os, idx);
  os.close();
  CUVS_EXPECTS(bool(os), "Error writing output %s", filename.c_str());
}

void serialize(cuvs::resources const& res, std::ostream& os, const index<int64_t>& idx)
{
  const auto& ix = *idx.impl();
  CUVS_EXPECTS(ix.centers.ptr != nullptr, "ivf_pq::serialize: the index holds no model");
  CUVS_EXPECTS(bool(os), "ivf_pq::serialize: the output stream is not writable");
  hipStream_t s = res.stream();

  write_scalar<int32_t>(os, "<i4", kSerializationVersion);
  write_scalar<int64_t>(os, "<i8", ix.size);
  write_scalar<uint32_t>(os, "<u4", ix.dim);
  write_scalar<uint32_t>(os, "<u4", ix.pq_bits);
  write_scalar<uint32_t>(os, "<u4", ix.pq_dim);
  write_scalar<uint8_t>(os, "|b1", ix.conservative_memory_allocation ? 1 : 0);
  write_scalar<int32_t>(os, "<i4", int32_t(ix.metric));
  write_scalar<int32_t>(os, "<i4", int32_t(ix.codebook_kind));
  write_scalar<int32_t>(os, "<i4", int32_t(list_layout::INTERLEAVED));
  write_scalar<uint32_t>(os, "<u4", ix.n_lists);

  auto dump = [&](const cuvs::device_buffer& b, const std::vector<uint64_t>& shape) {
    uint64_t n = 1;
    for (auto v : shape) { n *= v; }
    std::vector<float> h(n);
    CUVS_HIP_TRY(hipMemcpyAsync(h.data(), b.ptr, n * sizeof(float), hipMemcpyDeviceToHost, s));
    CUVS_HIP_TRY(hipStreamSynchronize(s));
    write_array(os, "<f4", shape, h.data(), n * sizeof(float));
  };
  const uint64_t n_books = ix.codebook_kind == codebook_gen::PER_SUBSPACE ? ix.pq_dim : ix.n_lists;
  dump(ix.pq_centers, {n_books, ix.pq_len, ix.book_size});
  dump(ix.centers, {ix.n_lists, ix.dim_ext});
  dump(ix.centers_rot, {ix.n_lists, ix.rot_dim});
  dump(ix.rotation, {ix.rot_dim, ix.dim});
  write_array(os, "<u4", {ix.n_lists}, ix.h_list_sizes.data(), sizeof(uint32_t) * ix.n_lists);

  // lists: the arenas hold them back to back in list order
  const uint64_t gb         = ix.group_bytes();
  const uint64_t total_rows = ix.h_row_offsets[ix.n_lists];
  std::vector<uint8_t> codes((total_rows / kIndexGroupSize) * gb);
  std::vector<int64_t> ids(total_rows);
  if (total_rows > 0) {
    CUVS_HIP_TRY(hipMemcpyAsync(codes.data(), ix.codes_arena.ptr, codes.size(), hipMemcpyDeviceToHost, s));
    CUVS_HIP_TRY(hipMemcpyAsync(ids.data(), ix.ids_arena.ptr, ids.size() * sizeof(int64_t),
                                hipMemcpyDeviceToHost, s));
    CUVS_HIP_TRY(hipStreamSynchronize(s));
  }
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    const uint32_t size = ix.h_list_sizes[l];
    write_scalar<uint32_t>(os, "<u4", size);
    if (size == 0) { continue; }
    const uint64_t groups = (uint64_t(size) + kIndexGroupSize - 1) / kIndexGroupSize;
    write_array(os, "|u1", {groups, ix.n_chunks, kIndexGroupSize, kIndexGroupVecLen},
                codes.data() + (ix.h_row_offsets[l] / kIndexGroupSize) * gb, groups * gb);
    write_array(os, "<i8", {size}, ids.data() + ix.h_row_offsets[l], uint64_t(size) * sizeof(int64_t));
  }
  CUVS_EXPECTS(bool(os), "ivf_pq::serialize: error writing to the output stream");
}

void deserialize(cuvs::resources const& res, const std::string& filename, index<int64_t>* idx)
{
  CUVS_EXPECTS(idx != nullptr, "index must not be null");
  std::ifstream is(filename, std::ios::in | std::ios::binary);
  CUVS_EXPECTS(bool(is), "Cannot open file %s", filename.c_str());
  deserialize(res, is, idx);
}

void deserialize(cuvs::resources const& res, std::istream& is, index<int64_t>* idx)
{
  CUVS_EXPECTS(idx != nullptr, "index must not be null");
  CUVS_EXPECTS(bool(is), "ivf_pq::deserialize: the input stream is not readable");

  const int ver = read_scalar<int32_t>(is, "version");
  CUVS_EXPECTS(ver == kSerializationVersion, "serialization version mismatch %d vs. %d", ver,
               kSerializationVersion);
  const int64_t n_rows = read_scalar<int64_t>(is, "size");
  index_params params;
  const uint32_t dim = read_scalar<uint32_t>(is, "dim");
  params.pq_bits     = read_scalar<uint32_t>(is, "pq_bits");
  params.pq_dim      = read_scalar<uint32_t>(is, "pq_dim");
  params.conservative_memory_allocation = read_scalar<uint8_t>(is, "conservative_memory_allocation") != 0;
  const int32_t metric = read_scalar<int32_t>(is, "metric");
  const int32_t kind   = read_scalar<int32_t>(is, "codebook_kind");
  const int32_t layout = read_scalar<int32_t>(is, "codes_layout");
  params.n_lists       = read_scalar<uint32_t>(is, "n_lists");
  CUVS_EXPECTS(kind == 0 || kind == 1, "ivf_pq::deserialize: invalid codebook_gen value %d", kind);
  CUVS_EXPECTS(layout == int32_t(list_layout::INTERLEAVED),
               "ivf_pq::deserialize: only the INTERLEAVED codes layout is supported (found %d)", layout);
  CUVS_EXPECTS(n_rows >= 0 && dim > 0 && params.pq_dim > 0 && params.n_lists > 0 &&
                 params.n_lists <= (1u << 30),
               "ivf_pq::deserialize: implausible header values");
  params.metric        = cuvs::distance::DistanceType(metric);
  params.codebook_kind = codebook_gen(kind);

  // derived dimensions through a scratch index, then the model tensors
  detail::index_impl dims;
  detail::init_index(dims, params, dim);
  const uint64_t n_books = params.codebook_kind == codebook_gen::PER_SUBSPACE ? dims.pq_dim : dims.n_lists;
  std::vector<float> pq_centers(n_books * dims.pq_len * dims.book_size);
  std::vector<float> centers(uint64_t(dims.n_lists) * dims.dim_ext);
  std::vector<float> centers_rot(uint64_t(dims.n_lists) * dims.rot_dim);
  std::vector<float> rotation(uint64_t(dims.rot_dim) * dims.dim);
  read_array(is, "pq_centers", 4, pq_centers.size(), pq_centers.data());
  read_array(is, "centers", 4, centers.size(), centers.data());
  read_array(is, "centers_rot", 4, centers_rot.size(), centers_rot.data());
  read_array(is, "rotation_matrix", 4, rotation.size(), rotation.data());
  std::vector<uint32_t> sizes(dims.n_lists);
  read_array(is, "list_sizes", 4, sizes.size(), sizes.data());

  index<int64_t> loaded = build(res, params, dim, pq_centers.data(), centers.data(),
                                centers_rot.data(), rotation.data());
  auto& ix = *loaded.impl();

  // lists into host images of the two arenas
  std::vector<uint64_t> offsets(ix.n_lists + 1, 0);
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    offsets[l + 1] = offsets[l] + cuvs::round_up_u64(sizes[l], kIndexGroupSize);
  }
  const uint64_t gb         = ix.group_bytes();
  const uint64_t total_rows = offsets[ix.n_lists];
  std::vector<uint8_t> codes((total_rows / kIndexGroupSize) * gb, 0);
  std::vector<int64_t> ids(total_rows, -1);
  uint64_t counted = 0;
  for (uint32_t l = 0; l < ix.n_lists; l++) {
    const std::string what = "list " + std::to_string(l);
    const uint32_t size    = read_scalar<uint32_t>(is, what + " size");
    CUVS_EXPECTS(size == sizes[l], "ivf_pq::deserialize: %s: size %u differs from list_sizes (%u)",
                 what.c_str(), size, sizes[l]);
    if (size == 0) { continue; }
    const uint64_t groups = (uint64_t(size) + kIndexGroupSize - 1) / kIndexGroupSize;
    read_array(is, what + " codes", 1, groups * gb, codes.data() + (offsets[l] / kIndexGroupSize) * gb);
    read_array(is, what + " indices", 8, size, ids.data() + offsets[l]);
    counted += size;
  }
  CUVS_EXPECTS(int64_t(counted) == n_rows, "ivf_pq::deserialize: list sizes add up to %llu, header says %lld",
               static_cast<unsigned long long>(counted), static_cast<long long>(n_rows));

  hipStream_t s = res.stream();
  // two groups of slack after the last list: scan kernels read whole 64-row tiles
  cuvs::device_buffer d_codes((total_rows / kIndexGroupSize + 2) * gb);
  cuvs::device_buffer d_ids(total_rows * sizeof(int64_t));
  CUVS_HIP_TRY(hipMemsetAsync(d_codes.ptr, 0, d_codes.bytes, s));
  if (total_rows > 0) {
    CUVS_HIP_TRY(hipMemcpyAsync(d_codes.ptr, codes.data(), codes.size(), hipMemcpyHostToDevice, s));
    CUVS_HIP_TRY(hipMemcpyAsync(d_ids.ptr, ids.data(), ids.size() * sizeof(int64_t), hipMemcpyHostToDevice, s));
  }
  CUVS_HIP_TRY(hipStreamSynchronize(s));
  ix.codes_arena   = std::move(d_codes);
  ix.ids_arena     = std::move(d_ids);
  ix.h_list_sizes  = sizes;
  ix.h_row_offsets = offsets;
  ix.recompute_internal_state(s);
  ix.rebuild_lead_plane(s);
  *idx = std::move(loaded);
}

}  // namespace cuvs::neighbors::ivf_pq
