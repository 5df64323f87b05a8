/*
 * Minimal stand-ins for the RAFT types that appear in the signatures of the cuVS C++ search API
 * (raft::resources, raft::device_matrix_view, raft::logic_error): a resources handle that owns a
 * HIP stream choice and a reusable device workspace, and non-owning row-major views.
 */
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace cuvs::memory {
class pool;     // sub-allocating device memory pool, internal to the library
class tracker;  // allocation tracking with a CSV reporter, internal to the library
}

// The library is built with hidden visibility; what this header declares is its C++ interface
// (the reference marks the same namespaces CUVS_EXPORT).
#pragma GCC visibility push(default)

namespace cuvs {

/** Error type thrown by every C++ entry point (role of raft::logic_error / RAFT_EXPECTS). */
struct logic_error : public std::runtime_error {
  explicit logic_error(const std::string& msg) : std::runtime_error(msg) {}
};

/** Non-owning row-major 2-D view (role of raft::device_matrix_view<T, int64_t, row_major>). */
template <typename T>
struct device_matrix_view {
  T* data      = nullptr;
  int64_t rows = 0;
  int64_t cols = 0;
  T* data_handle() const { return data; }
  int64_t extent(int i) const { return i == 0 ? rows : cols; }
};

template <typename T>
device_matrix_view<T> make_device_matrix_view(T* data, int64_t rows, int64_t cols)
{
  return device_matrix_view<T>{data, rows, cols};
}

/** Non-owning row-major 2-D view of host memory (role of raft::host_matrix_view<T, int64_t, row_major>). */
template <typename T>
struct host_matrix_view {
  T* data      = nullptr;
  int64_t rows = 0;
  int64_t cols = 0;
  T* data_handle() const { return data; }
  int64_t extent(int i) const { return i == 0 ? rows : cols; }
};

template <typename T>
host_matrix_view<T> make_host_matrix_view(T* data, int64_t rows, int64_t cols)
{
  return host_matrix_view<T>{data, rows, cols};
}

/** Non-owning 1-D view (role of raft::device_vector_view<T, uint32_t>). */
template <typename T>
struct device_vector_view {
  T* data      = nullptr;
  int64_t size = 0;
  T* data_handle() const { return data; }
  int64_t extent(int) const { return size; }
};

template <typename T>
device_vector_view<T> make_device_vector_view(T* data, int64_t size)
{
  return device_vector_view<T>{data, size};
}

/** Per-stage timing of a search (filled when profiling is enabled on the resources). */
/** The kernel that scanned the pairs of a search in full (search_profile::scan_kernel). */
enum scan_kernel_id : uint32_t {
  scan_kernel_generic     = 0,
  scan_kernel_stream      = 1,
  scan_kernel_fast        = 2,
  scan_kernel_direct      = 3,
  scan_kernel_nibble      = 4,
  scan_kernel_nibble_pack = 5,
  scan_kernel_slab        = 6,
};

struct search_profile {
  uint32_t n_queries       = 0;
  uint32_t n_probes        = 0;
  uint32_t k               = 0;
  uint32_t n_scan_launches = 0;
  float coarse_ms          = 0;
  float rotate_ms          = 0;
  float scan_ms            = 0;
  float merge_ms           = 0;
  float total_ms           = 0;
  uint64_t scan_bytes      = 0;
  uint64_t scan_rows       = 0;
  // L2 early stop: the scan stage split into its three launches (zero when not used)
  float lead_scan_ms         = 0;
  float screen_ms            = 0;
  float survivor_scan_ms     = 0;
  uint32_t scan_kernel       = 0;  // scan_kernel_id of the last batch
  uint64_t lead_bytes        = 0;
  uint64_t screen_bytes      = 0;
  uint64_t survivor_bytes    = 0;
  uint64_t n_screened_pairs  = 0;
  uint64_t n_surviving_pairs = 0;
  uint64_t n_far_pairs       = 0;  // screened pairs dropped on the length of their residual alone
};

/** Choices the search otherwise makes by itself, for measurements and tests that compare the
 *  library's code paths with each other.  None of them changes a result. */
struct search_tuning {
  /** L2 early stop (leading lists in full, the others screened, survivors in full):
   *  0 = the library decides per batch, 1 = never: every probed list is scanned in full,
   *  2 = whenever the kernels support the search's parameters. */
  int early_stop = 0;
  /** Every search goes through the generic scan kernel. */
  bool generic_scan = false;
  /** Coarse search by the fp32 contraction and selection instead of the two-precision selection. */
  bool plain_coarse = false;
  /** The internal batches of a search run one after the other on the handle's stream instead of
   *  side by side on streams of the handle's own. */
  bool serial_batches = false;
};

/**
 * One stream plus a cached device workspace (role of raft::resources with a workspace memory
 * resource).  Not thread-safe: use one handle per host thread; an index may be shared.
 */
class resources {
 public:
  resources();
  ~resources();
  resources(const resources&)            = delete;
  resources& operator=(const resources&) = delete;

  hipStream_t stream() const { return stream_; }
  /**
   * Work the library queues from now on goes to `s`.  The cached workspace is shared by
   * consecutive calls: when the stream changes while work queued on the previous one may still use
   * it, the new stream is made to wait for that work first (an event recorded on the previous
   * stream), so calls on the same handle stay ordered across the switch.
   */
  void set_stream(hipStream_t s);
  void sync() const;
  int device_id() const { return device_; }

  /** Upper bound for the cached workspace in bytes (0 = no explicit bound). */
  void set_workspace_limit(size_t bytes) { workspace_limit_ = bytes; }
  size_t workspace_limit() const { return workspace_limit_; }

  /**
   * Give this handle a device memory pool of its own, reserved up front and growing on demand
   * (role of raft::resource::set_workspace_resource with an rmm pool_memory_resource): the cached
   * workspace and the C API's cuvsRMMAlloc / cuvsRMMFree on this handle then come out of it.
   */
  void set_workspace_pool(size_t initial_bytes);
  memory::pool* workspace_pool() const { return pool_.get(); }

  /**
   * From now until this handle is destroyed, every allocation and release the library makes is
   * counted and sampled into a CSV file by a background thread (role of
   * raft::memory_tracking_resources).  One tracking handle per process at a time.
   */
  void track_memory(const char* csv_path, int64_t sample_interval_ms);

  /** Bump allocation out of the cached workspace; valid until the next reset_workspace(). */
  void* workspace_alloc(size_t bytes);
  /** Make sure the workspace can serve `bytes` in total before the first allocation of a call. */
  void reserve_workspace(size_t bytes);
  void reset_workspace() { workspace_used_ = 0; }
  size_t workspace_capacity() const { return workspace_capacity_; }
  /**
   * Serve the workspace from `bytes` of device memory that somebody else owns (256-byte aligned)
   * from now on: the handle then never allocates or frees device memory for it, and a call that
   * needs more fails instead of growing it.  For handles that have no workspace yet.
   */
  void borrow_workspace(void* ptr, size_t bytes);
  bool workspace_borrowed() const { return workspace_borrowed_; }

  /**
   * Handle number `i` of this handle's own: another stream (default priority) and another cached
   * workspace, for internal batches of one call that run beside each other.  Created on first
   * use, destroyed with this handle; null if the stream cannot be made.  fork(): work queued on
   * the side streams from now on starts after what this handle's stream holds now; join(): this
   * handle's stream continues after what the side streams hold now.
   */
  static constexpr int kMaxSideHandles = 3;
  resources* side(int i);
  void fork_sides(int n);
  void join_sides(int n);

  search_tuning tuning;
  bool profiling = false;
  struct profile_state;
  profile_state* prof = nullptr;  // lazily created event set
  search_profile last_profile;

 private:
  int device_             = 0;
  hipStream_t stream_     = nullptr;
  void* workspace_        = nullptr;
  size_t workspace_capacity_ = 0;
  size_t workspace_used_  = 0;
  size_t workspace_limit_ = 0;
  // workspaces outgrown after a call was captured into a HIP graph while they were current: the
  // graph keeps their addresses, so they stay allocated until the handle goes
  std::vector<void*> retired_;
  std::vector<bool> retired_pooled_;
  bool workspace_captured_ = false;  // a call ran under stream capture on the current workspace
  hipEvent_t order_event_  = nullptr;  // set_stream: orders the new stream after the previous one
  std::shared_ptr<memory::pool> pool_;  // set_workspace_pool
  bool workspace_pooled_ = false;       // workspace_ came out of pool_
  bool workspace_borrowed_ = false;     // workspace_ belongs to the caller of borrow_workspace
  void release_workspace();
  memory::tracker* tracker_ = nullptr;  // track_memory
  struct side_handle {
    resources* handle  = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t done    = nullptr;
  };
  side_handle sides_[kMaxSideHandles];
  hipEvent_t fork_event_ = nullptr;
};

}  // namespace cuvs

#pragma GCC visibility pop
