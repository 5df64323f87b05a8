/* Instances of the slab scan kernel (scan_slab.cuh) for pq_len = 1. */
#include "scan_slab.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

bool launch_scan_slab_len1(const scan_args& a, hipStream_t stream) { return launch_slab_len<1>(a, stream); }

}  // namespace cuvs::neighbors::ivf_pq::detail
