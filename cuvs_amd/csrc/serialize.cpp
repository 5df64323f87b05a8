/*
 * Index (de)serialisation entry points.  The cuVS on-disk format
 * (cpp/src/neighbors/ivf_pq/ivf_pq_serialize.cuh:41-87,124-211) frames every field with RAFT's
 * NumPy-style mdspan serializer, whose source is not part of the cuVS tree; until that framing is
 * restated and pinned these calls fail loudly instead of writing an incompatible file.
 */
#include "detail.hpp"

namespace cuvs::neighbors::ivf_pq {

void serialize(cuvs::resources const&, const std::string& filename, const index<int64_t>&)
{
  fail("ivf_pq::serialize(%s): the cuVS index file format is not implemented in this library yet",
       filename.c_str());
}

void deserialize(cuvs::resources const&, const std::string& filename, index<int64_t>*)
{
  fail("ivf_pq::deserialize(%s): the cuVS index file format is not implemented in this library yet",
       filename.c_str());
}

}  // namespace cuvs::neighbors::ivf_pq
