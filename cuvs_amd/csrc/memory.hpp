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

/** rmm::percent_of_free_device_memory: that share of the free memory, a multiple of 256 bytes. */
size_t percent_of_free_device_memory(int percent);

}  // namespace cuvs::memory
