/*
 * cuvs::resources: stream choice plus a cached device workspace that grows on demand and is
 * reused by consecutive calls (role of raft::resources with a workspace memory resource).
 */
#include "detail.hpp"

namespace cuvs {

resources::resources()
{
  CUVS_HIP_TRY(hipGetDevice(&device_));
}

resources::~resources()
{
  if (workspace_ != nullptr) { (void)hipFree(workspace_); }
  for (void* p : retired_) { (void)hipFree(p); }
  extern void destroy_profile_state(resources::profile_state*);
  destroy_profile_state(prof);
}

void resources::sync() const { CUVS_HIP_TRY(hipStreamSynchronize(stream_)); }

void resources::reserve_workspace(size_t bytes)
{
  if (bytes <= workspace_capacity_) { return; }
  CUVS_EXPECTS(workspace_used_ == 0, "workspace cannot grow while allocations are live");
  // work queued earlier may still read the old block: wait, then release it
  CUVS_HIP_TRY(hipStreamSynchronize(stream_));
  if (workspace_ != nullptr) { CUVS_HIP_TRY(hipFree(workspace_)); }
  workspace_          = nullptr;
  workspace_capacity_ = 0;
  const size_t want   = round_up_u64(bytes + bytes / 8, size_t(1) << 20);
  CUVS_HIP_TRY(hipMalloc(&workspace_, want));
  workspace_capacity_ = want;
}

void* resources::workspace_alloc(size_t bytes)
{
  const size_t aligned = round_up_u64(bytes == 0 ? 1 : bytes, 256);
  CUVS_EXPECTS(workspace_used_ + aligned <= workspace_capacity_,
               "workspace exhausted: %zu + %zu > %zu (reserve_workspace was too small)",
               workspace_used_, aligned, workspace_capacity_);
  void* p = static_cast<char*>(workspace_) + workspace_used_;
  workspace_used_ += aligned;
  return p;
}

}  // namespace cuvs
