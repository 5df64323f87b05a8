/*
 * Which searches the slab scan kernel (scan_slab.cuh) takes, and its launch by pq_len (the
 * instances of each pq_len are a translation unit of their own, scan_slab_len*.hip).
 */
#include "scan_slab.cuh"

namespace cuvs::neighbors::ivf_pq::detail {

bool launch_scan_slab_len1(const scan_args& a, hipStream_t stream);
bool launch_scan_slab_len2(const scan_args& a, hipStream_t stream);
bool launch_scan_slab_len3(const scan_args& a, hipStream_t stream);
bool launch_scan_slab_len4(const scan_args& a, hipStream_t stream);
bool launch_scan_slab_len8(const scan_args& a, hipStream_t stream);

uint32_t scan_slab_keys_per_pair(const scan_args& a)
{
  if (!a.fused || a.pq_bits != 8 || a.k > kSlabMaxK) { return 0; }
  if (a.rot_dim != a.pq_dim * a.pq_len) { return 0; }
  if (a.lut_dtype != CUDA_R_16F && a.lut_dtype != CUDA_R_8U && !(a.lut_dtype == CUDA_R_32F && !a.out_half)) { return 0; }
  if (a.pq_dim < 32 || a.pq_dim % 32 != 0) { return 0; }
  const bool len = a.pq_len == 1 || a.pq_len == 2 || a.pq_len == 3 || a.pq_len == 4 || a.pq_len == 8;
  return len ? kSlabWG * a.k : 0;
}

bool launch_scan_slab(const scan_args& a, hipStream_t stream)
{
  if (scan_slab_keys_per_pair(a) == 0 || a.n_queries == 0 || a.desc == nullptr) { return false; }
  switch (a.pq_len) {
    case 1: return launch_scan_slab_len1(a, stream);
    case 2: return launch_scan_slab_len2(a, stream);
    case 3: return launch_scan_slab_len3(a, stream);
    case 4: return launch_scan_slab_len4(a, stream);
    case 8: return launch_scan_slab_len8(a, stream);
    default: return false;
  }
}

}  // namespace cuvs::neighbors::ivf_pq::detail
