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

resources* resources::side(int i)
{
  if (i < 0 || i >= kMaxSideHandles) { return nullptr; }
  side_handle& sh = sides_[i];
  if (sh.handle == nullptr) {
    hipStream_t st = nullptr;
    hipEvent_t ev  = nullptr;
    if (hipStreamCreateWithFlags(&st, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      if (st != nullptr) { (void)hipStreamDestroy(st); }
      return nullptr;
    }
    sh.stream = st;
    sh.done   = ev;
    sh.handle = new resources();
    sh.handle->set_stream(st);
  }
  sh.handle->tuning           = tuning;
  sh.handle->workspace_limit_ = workspace_limit_;
  return sh.handle;
}

void resources::fork_sides(int n)
{
  if (fork_event_ == nullptr) { CUVS_HIP_TRY(hipEventCreateWithFlags(&fork_event_, hipEventDisableTiming)); }
  CUVS_HIP_TRY(hipEventRecord(fork_event_, stream_));
  for (int i = 0; i < n && i < kMaxSideHandles; i++) {
    if (sides_[i].handle != nullptr) { CUVS_HIP_TRY(hipStreamWaitEvent(sides_[i].stream, fork_event_, 0)); }
  }
}

void resources::join_sides(int n)
{
  for (int i = 0; i < n && i < kMaxSideHandles; i++) {
    if (sides_[i].handle == nullptr) { continue; }
    CUVS_HIP_TRY(hipEventRecord(sides_[i].done, sides_[i].stream));
    CUVS_HIP_TRY(hipStreamWaitEvent(stream_, sides_[i].done, 0));
  }
}

resources::~resources()
{
  for (side_handle& sh : sides_) {
    if (sh.handle == nullptr) { continue; }
    (void)hipStreamSynchronize(sh.stream);
    delete sh.handle;  // its workspace
    (void)hipEventDestroy(sh.done);
    (void)hipStreamDestroy(sh.stream);
  }
  if (fork_event_ != nullptr) { (void)hipEventDestroy(fork_event_); }
  // a pool of this handle's own returns everything it holds when it goes, right after this body
  if (!(workspace_pooled_ && pool_)) { release_workspace(); }
  for (size_t i = 0; i < retired_.size(); i++) {
    if (!(retired_pooled_[i] && pool_)) { memory::deallocate(retired_[i]); }  // the pool frees its own
  }
  if (order_event_ != nullptr) { (void)hipEventDestroy(order_event_); }
  extern void destroy_profile_state(resources::profile_state*);
  destroy_profile_state(prof);
  if (tracker_ != nullptr) {
    // the handle's own pool goes after this body: what it still holds counts as live in the last row
    memory::stop_tracking(tracker_);
  }
}

void resources::track_memory(const char* csv_path, int64_t sample_interval_ms)
{
  CUVS_EXPECTS(tracker_ == nullptr, "this handle tracks memory already");
  tracker_ = memory::start_tracking(csv_path, sample_interval_ms);
}

void resources::sync() const { CUVS_HIP_TRY(hipStreamSynchronize(stream_)); }

void resources::set_stream(hipStream_t s)
{
  if (s == stream_) { return; }
  const hipStream_t prev = stream_;
  stream_                = s;
  if (workspace_ == nullptr || workspace_borrowed_) { return; }
  // Under stream capture neither an event query nor a dependency on work outside the graph is
  // allowed (either would invalidate the capture): a caller that switches a handle to or from a
  // capturing stream orders the two streams itself.
  for (hipStream_t each : {prev, s}) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(each, &st) != hipSuccess) {
      (void)hipGetLastError();  // a stream that no longer exists
      if (each == s) { return; }
      continue;
    }
    if (st != hipStreamCaptureStatusNone) { return; }
  }
  // Whatever the previous stream still has queued may read or write the workspace.  The previous
  // stream may be gone by now (a caller that makes a stream per request): then its work is done
  // and the failing record is ignored.
  if (order_event_ == nullptr &&
      hipEventCreateWithFlags(&order_event_, hipEventDisableTiming) != hipSuccess) {
    (void)hipGetLastError();
    order_event_ = nullptr;
    return;
  }
  if (hipEventRecord(order_event_, prev) != hipSuccess) {
    (void)hipGetLastError();
    return;
  }
  if (hipEventQuery(order_event_) == hipSuccess) { return; }  // nothing pending: no dependency needed
  (void)hipGetLastError();                                     // hipErrorNotReady is not an error here
  CUVS_HIP_TRY(hipStreamWaitEvent(s, order_event_, 0));
}

void resources::borrow_workspace(void* ptr, size_t bytes)
{
  CUVS_EXPECTS(workspace_ == nullptr && workspace_used_ == 0,
               "a handle that already caches a workspace cannot borrow one");
  CUVS_EXPECTS(ptr != nullptr && reinterpret_cast<uintptr_t>(ptr) % 256 == 0,
               "a borrowed workspace must be 256-byte aligned device memory");
  workspace_          = ptr;
  workspace_capacity_ = bytes;
  workspace_borrowed_ = true;
}

void resources::release_workspace()
{
  if (workspace_ == nullptr) { return; }
  void* p             = workspace_;
  workspace_          = nullptr;
  workspace_capacity_ = 0;
  if (workspace_borrowed_) {
    workspace_borrowed_ = false;
    return;
  }
  if (workspace_pooled_ && pool_) {
    (void)memory::pool_deallocate(*pool_, p, stream_, true);
  } else {
    memory::deallocate(p);
  }
}

void resources::set_workspace_pool(size_t initial_bytes)
{
  CUVS_EXPECTS(workspace_used_ == 0, "the workspace pool cannot change while allocations are live");
  size_t own = (workspace_pooled_ && workspace_ != nullptr) ? 1 : 0;
  for (bool pooled : retired_pooled_) { own += pooled ? 1 : 0; }
  CUVS_EXPECTS(!pool_ || memory::pool_live_allocations(*pool_) == own,
               "the previous workspace pool still has live allocations");
  auto next = memory::make_pool(initial_bytes, 0, false);
  CUVS_HIP_TRY(hipStreamSynchronize(stream_));
  release_workspace();
  // workspaces kept for captured graphs go back with the pool they came from (such graphs must
  // not be replayed after the pool changes)
  for (size_t i = 0; i < retired_.size(); i++) {
    if (retired_pooled_[i] && pool_) {
      (void)memory::pool_deallocate(*pool_, retired_[i], stream_, true);
      retired_[i] = nullptr;
    }
  }
  {
    std::vector<void*> keep;
    for (void* p : retired_) {
      if (p != nullptr) { keep.push_back(p); }
    }
    retired_ = std::move(keep);
    retired_pooled_.assign(retired_.size(), false);
  }
  pool_ = std::move(next);
}

void resources::reserve_workspace(size_t bytes)
{
  if (!workspace_captured_ && workspace_ != nullptr && !workspace_borrowed_) {
    // a call recorded into a HIP graph keeps the workspace's address for its replays
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream_, &st) == hipSuccess) {
      workspace_captured_ = st != hipStreamCaptureStatusNone;
    } else {
      (void)hipGetLastError();
    }
  }
  if (bytes <= workspace_capacity_) { return; }
  CUVS_EXPECTS(!workspace_borrowed_,
               "this call needs %zu bytes of workspace, more than the %zu bytes the handle borrowed",
               bytes, workspace_capacity_);
  CUVS_EXPECTS(workspace_used_ == 0, "workspace cannot grow while allocations are live");
  // work queued earlier may still read the old block: wait, then release it
  CUVS_HIP_TRY(hipStreamSynchronize(stream_));
  if (workspace_captured_ && workspace_ != nullptr) {
    retired_.push_back(workspace_);
    retired_pooled_.push_back(workspace_pooled_);
    workspace_          = nullptr;
    workspace_capacity_ = 0;
    workspace_captured_ = false;
  } else {
    release_workspace();
  }
  const size_t want = round_up_u64(bytes + bytes / 8, size_t(1) << 20);
  if (pool_) {
    workspace_        = memory::pool_allocate(*pool_, want, stream_, true);
    workspace_pooled_ = true;
  } else {
    workspace_        = memory::allocate(want);
    workspace_pooled_ = false;
  }
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
