/*
 * Where the library's device memory comes from (role of rmm's current device resource and of
 * rmm::mr::pool_memory_resource / cuda_async_memory_resource behind cuvsRMMAlloc,
 * c/src/core/c_api.cpp:167-216): plain hipMalloc by default, a sub-allocating pool or the
 * runtime's stream-ordered allocator when a caller switches the process over.
 */
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <memory>

namespace cuvs::memory {

/**
 * Best-fit sub-allocator over a few large upstream blocks.  Freed ranges go back to the pool
 * (never to the device) and merge with free neighbours; a range freed in stream order carries an
 * event that a later owner on another stream waits for, so no call synchronises the device.
 * Thread-safe.
 */
class pool;

/** `maximum` == 0: the pool may grow until the device is full. */
std::shared_ptr<pool> make_pool(size_t initial_bytes, size_t maximum_bytes, bool managed);
/** `ordered`: the caller uses the range on `stream` only after this call, in stream order. */
void* pool_allocate(pool& p, size_t bytes, hipStream_t stream, bool ordered);
/** False when `ptr` is not one of this pool's live ranges' addresses. */
bool pool_deallocate(pool& p, void* ptr, hipStream_t stream, bool ordered);
size_t pool_reserved_bytes(const pool& p);
size_t pool_live_allocations(const pool& p);

/** Library-internal allocations: usable by any stream on return; release waits for the device
 *  like hipFree does. */
void* allocate(size_t bytes);
void deallocate(void* ptr) noexcept;

/** Stream-ordered allocations of the C API. */
void* allocate_on_stream(size_t bytes, hipStream_t stream);
void deallocate_on_stream(void* ptr, hipStream_t stream);

/** Process-wide switches (cuvsRMMPoolMemoryResourceEnable / AsyncMemoryResourceEnable / Reset).
 *  Memory handed out earlier stays valid and is released through the resource it came from. */
void enable_pool(int initial_percent, int maximum_percent, bool managed);
void enable_async();
void reset();

/** Pinned host memory (cuvsRMMHostAlloc / cuvsRMMHostFree). */
void* host_allocate(size_t bytes);
void host_deallocate(void* ptr);

/**
 * Allocation tracking (role of raft::memory_tracking_resources behind
 * cuvsResourcesCreateWithMemoryTracking, c/src/core/c_api.cpp:57-72): while a tracker is alive every
 * allocation and release made through this file is counted, and a background thread writes samples
 * to a CSV file: the header at once, then one row after each burst of activity, not more often
 * than every `interval_ms`, each flushed as written, and a last row when tracking stops.
 * Columns: elapsed_ms, device_current_bytes, device_peak_bytes, pinned_current_bytes,
 * pinned_peak_bytes, allocations, deallocations.  One tracker per process at a time.
 */
class tracker;
tracker* start_tracking(const char* csv_path, int64_t interval_ms);
void stop_tracking(tracker* t) noexcept;

/** rmm::percent_of_free_device_memory: that share of the free memory, a multiple of 256 bytes. */
size_t percent_of_free_device_memory(int percent);

}  // namespace cuvs::memory
