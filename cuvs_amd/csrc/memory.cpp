/*
 * Device memory sources: plain hipMalloc, a sub-allocating pool, or the runtime's stream-ordered
 * allocator, switchable for the whole process like rmm's current device resource
 * (c/src/core/c_api.cpp:185-216).
 */
#include "detail.hpp"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <thread>
#include <unordered_map>
#include <unordered_set>
#include <utility>
#include <vector>

namespace cuvs::memory {

namespace {
constexpr size_t kGranule     = 256;                // every range is a multiple of this, and aligned to it
constexpr size_t kUpstreamPad = size_t(2) << 20;    // upstream blocks are multiples of this
constexpr size_t kFirstGrowth = size_t(64) << 20;   // an empty pool grows by at least this much
constexpr size_t kMaxFences   = 8;                  // finished fences are dropped beyond this many

/** Marks the point in a stream after which a freed range may be reused. */
struct fence {
  hipEvent_t event   = nullptr;
  hipStream_t stream = nullptr;
  fence(hipStream_t s) : stream(s)
  {
    CUVS_HIP_TRY(hipEventCreateWithFlags(&event, hipEventDisableTiming));
    hipError_t st = hipEventRecord(event, s);
    if (st != hipSuccess) {
      (void)hipEventDestroy(event);
      fail("hipEventRecord failed while freeing pooled memory: %s", hipGetErrorString(st));
    }
  }
  ~fence() { (void)hipEventDestroy(event); }
  fence(const fence&)            = delete;
  fence& operator=(const fence&) = delete;
};
using fence_list = std::vector<std::shared_ptr<fence>>;

void merge_fences(fence_list& into, const fence_list& from)
{
  for (const auto& f : from) {
    if (std::find(into.begin(), into.end(), f) == into.end()) { into.push_back(f); }
  }
  if (into.size() > kMaxFences) {
    into.erase(std::remove_if(into.begin(), into.end(),
                              [](const std::shared_ptr<fence>& f) {
                                return hipEventQuery(f->event) == hipSuccess;
                              }),
               into.end());
  }
}
}  // namespace

/* ---------------------------------------------------------------------------------------- */
/* allocation tracking                                                                       */
/* ---------------------------------------------------------------------------------------- */

enum class space { device = 0, pinned = 1 };

class tracker {
 public:
  tracker(const char* csv_path, int64_t interval_ms)
    : interval_(interval_ms), start_(std::chrono::steady_clock::now())
  {
    file_ = std::fopen(csv_path, "w");
    CUVS_EXPECTS(file_ != nullptr, "cannot open %s for writing", csv_path);
    std::fputs("elapsed_ms,device_current_bytes,device_peak_bytes,pinned_current_bytes,pinned_peak_bytes,"
               "allocations,deallocations\n",
               file_);
    std::fflush(file_);
    sampler_ = std::thread([this] { run(); });
  }

  ~tracker()
  {
    {
      std::lock_guard<std::mutex> lock(mutex_);
      stop_ = true;
    }
    wake_.notify_all();
    if (sampler_.joinable()) { sampler_.join(); }
    write_row();  // the state at the end, whatever the sampler saw last
    std::fclose(file_);
  }

  void allocated(void* ptr, size_t bytes, space where)
  {
    std::lock_guard<std::mutex> lock(mutex_);
    live_[ptr] = {bytes, where};
    auto& u    = usage_[int(where)];
    u.current += bytes;
    u.peak = std::max(u.peak, u.current);
    n_alloc_ += 1;
    dirty_ = true;
    wake_.notify_all();
  }

  /** Ranges handed out before tracking began are not known here and pass unnoticed. */
  void released(void* ptr)
  {
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = live_.find(ptr);
    if (it == live_.end()) { return; }
    usage_[int(it->second.second)].current -= it->second.first;
    live_.erase(it);
    n_free_ += 1;
    dirty_ = true;
    wake_.notify_all();
  }

 private:
  struct usage {
    size_t current = 0, peak = 0;
  };

  void run()
  {
    std::unique_lock<std::mutex> lock(mutex_);
    while (!stop_) {
      wake_.wait(lock, [this] { return dirty_ || stop_; });
      if (stop_) { break; }
      dirty_ = false;
      lock.unlock();
      write_row();
      lock.lock();
      // the interval is the least time between two rows; a stop request ends the wait
      wake_.wait_for(lock, std::chrono::milliseconds(interval_), [this] { return stop_; });
    }
  }

  void write_row()
  {
    usage dev, pin;
    uint64_t n_alloc, n_free;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      dev     = usage_[0];
      pin     = usage_[1];
      n_alloc = n_alloc_;
      n_free  = n_free_;
    }
    const double ms =
      std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - start_).count();
    std::lock_guard<std::mutex> lock(file_mutex_);
    std::fprintf(file_, "%.3f,%zu,%zu,%zu,%zu,%llu,%llu\n", ms, dev.current, dev.peak, pin.current, pin.peak,
                 static_cast<unsigned long long>(n_alloc), static_cast<unsigned long long>(n_free));
    std::fflush(file_);
  }

  int64_t interval_;
  std::chrono::steady_clock::time_point start_;
  std::FILE* file_ = nullptr;
  std::mutex mutex_, file_mutex_;
  std::condition_variable wake_;
  std::thread sampler_;
  bool stop_ = false, dirty_ = false;
  usage usage_[2];
  uint64_t n_alloc_ = 0, n_free_ = 0;
  std::unordered_map<void*, std::pair<size_t, space>> live_;
};

namespace {
std::atomic<tracker*> g_tracker{nullptr};

inline void note_allocated(void* ptr, size_t bytes, space where = space::device)
{
  if (tracker* t = g_tracker.load(std::memory_order_acquire)) { t->allocated(ptr, bytes, where); }
}
inline void note_released(void* ptr)
{
  if (tracker* t = g_tracker.load(std::memory_order_acquire)) { t->released(ptr); }
}
}  // namespace

tracker* start_tracking(const char* csv_path, int64_t interval_ms)
{
  CUVS_EXPECTS(csv_path != nullptr && csv_path[0] != '\0', "csv_path must be a non-empty string");
  CUVS_EXPECTS(interval_ms >= 0, "sample_interval_ms must be >= 0");
  auto* t            = new tracker(csv_path, interval_ms);
  tracker* expected  = nullptr;
  if (!g_tracker.compare_exchange_strong(expected, t)) {
    delete t;
    fail("memory tracking is already active in this process: one tracking handle at a time");
  }
  return t;
}

void stop_tracking(tracker* t) noexcept
{
  if (t == nullptr) { return; }
  tracker* expected = t;
  g_tracker.compare_exchange_strong(expected, nullptr);
  delete t;
}

class pool {
 public:
  pool(size_t initial_bytes, size_t maximum_bytes, bool managed)
    : maximum_(maximum_bytes), managed_(managed)
  {
    CUVS_HIP_TRY(hipGetDevice(&device_));
    CUVS_EXPECTS(maximum_ == 0 || initial_bytes <= maximum_,
                 "the initial pool size (%zu) exceeds the maximum pool size (%zu)", initial_bytes,
                 maximum_);
    if (initial_bytes > 0) {
      std::lock_guard<std::mutex> lock(mutex_);
      add_upstream_block(round_up_u64(initial_bytes, kUpstreamPad), initial_bytes);
    }
  }

  ~pool()
  {
    for (auto& b : upstream_) { (void)hipFree(b.first); }
  }

  void* allocate(size_t bytes, hipStream_t stream, bool ordered)
  {
    const size_t size = round_up_u64(bytes == 0 ? 1 : bytes, kGranule);
    fence_list waits;
    char* addr = nullptr;
    {
      std::lock_guard<std::mutex> lock(mutex_);
      auto it = free_.lower_bound({size, nullptr});
      if (it == free_.end()) {
        grow(size);
        it = free_.lower_bound({size, nullptr});
      }
      addr = it->second;
      free_.erase(it);
      range& r = ranges_.at(addr);
      if (r.bytes - size >= kGranule) {
        range rest;
        rest.bytes  = r.bytes - size;
        rest.free   = true;
        rest.head   = false;
        rest.fences = r.fences;
        ranges_.emplace(addr + size, std::move(rest));
        free_.insert({r.bytes - size, addr + size});
        r.bytes = size;
      }
      r.free = false;
      waits.swap(r.fences);
      live_ += 1;
    }
    for (const auto& f : waits) {
      if (ordered && f->stream == stream) { continue; }  // already ordered behind the release
      hipError_t st = ordered ? hipStreamWaitEvent(stream, f->event, 0) : hipEventSynchronize(f->event);
      if (st != hipSuccess) {
        // give the range back, still fenced, before reporting
        std::lock_guard<std::mutex> lock(mutex_);
        release_locked(addr, waits);
        fail("waiting for the previous owner of pooled memory failed: %s", hipGetErrorString(st));
      }
    }
    note_allocated(addr, size);
    return addr;
  }

  bool deallocate(void* ptr, hipStream_t stream, bool ordered)
  {
    if (!owns(ptr)) { return false; }
    fence_list marks;
    if (ordered) {
      marks.push_back(std::make_shared<fence>(stream));
    } else {
      // the caller does not say which stream used the range last: wait for all of them
      CUVS_HIP_TRY(hipDeviceSynchronize());
    }
    note_released(ptr);
    std::lock_guard<std::mutex> lock(mutex_);
    return release_locked(static_cast<char*>(ptr), marks);
  }

  /** True when `ptr` is the address of a live range of this pool. */
  bool owns(const void* ptr) const
  {
    std::lock_guard<std::mutex> lock(mutex_);
    auto it = ranges_.find(static_cast<char*>(const_cast<void*>(ptr)));
    return it != ranges_.end() && !it->second.free;
  }

  size_t reserved_bytes() const
  {
    std::lock_guard<std::mutex> lock(mutex_);
    return reserved_;
  }

  size_t live_allocations() const
  {
    std::lock_guard<std::mutex> lock(mutex_);
    return live_;
  }

 private:
  struct range {
    size_t bytes = 0;
    bool free    = true;
    bool head    = false;  // first range of an upstream block: never merged into its predecessor
    fence_list fences;     // what the next owner has to wait for
  };

  bool release_locked(char* addr, const fence_list& marks)
  {
    auto it = ranges_.find(addr);
    if (it == ranges_.end() || it->second.free) { return false; }
    it->second.free   = true;
    it->second.fences = marks;
    auto next = std::next(it);
    if (next != ranges_.end() && next->second.free && !next->second.head &&
        next->first == addr + it->second.bytes) {
      free_.erase({next->second.bytes, next->first});
      it->second.bytes += next->second.bytes;
      merge_fences(it->second.fences, next->second.fences);
      ranges_.erase(next);
    }
    if (!it->second.head && it != ranges_.begin()) {
      auto prev = std::prev(it);
      if (prev->second.free && prev->first + prev->second.bytes == addr) {
        free_.erase({prev->second.bytes, prev->first});
        prev->second.bytes += it->second.bytes;
        merge_fences(prev->second.fences, it->second.fences);
        ranges_.erase(it);
        it = prev;
      }
    }
    free_.insert({it->second.bytes, it->first});
    live_ -= 1;
    return true;
  }

  void grow(size_t size)
  {
    const size_t room = maximum_ == 0 ? ~size_t(0) : maximum_ - std::min(maximum_, reserved_);
    CUVS_EXPECTS(size <= room,
                 "memory pool exhausted: %zu more bytes asked for, %zu reserved, maximum %zu", size,
                 reserved_, maximum_);
    size_t want = std::max(size, std::max(reserved_, kFirstGrowth));
    want        = round_up_u64(want, kUpstreamPad);
    if (want > room) { want = room / kGranule * kGranule; }
    if (want < size || !try_upstream_block(want)) {
      // the device may still have room for just this request
      if (!try_upstream_block(round_up_u64(size, kGranule))) {
        fail("memory pool cannot grow by %zu bytes: the device is out of memory (%zu reserved)", size,
             reserved_);
      }
    }
  }

  bool try_upstream_block(size_t bytes)
  {
    void* p       = nullptr;
    hipError_t st = managed_ ? hipMallocManaged(&p, bytes, hipMemAttachGlobal) : hipMalloc(&p, bytes);
    if (st != hipSuccess) {
      (void)hipGetLastError();  // the failure is handled here: do not leave it for the next call
      return false;
    }
    upstream_.push_back({p, bytes});
    reserved_ += bytes;
    range r;
    r.bytes = bytes;
    r.free  = true;
    r.head  = true;
    ranges_.emplace(static_cast<char*>(p), std::move(r));
    free_.insert({bytes, static_cast<char*>(p)});
    return true;
  }

  void add_upstream_block(size_t bytes, size_t asked)
  {
    if (!try_upstream_block(bytes)) {
      fail("cannot reserve %zu bytes of %s memory for the pool", asked, managed_ ? "managed" : "device");
    }
  }

  mutable std::mutex mutex_;
  std::map<char*, range> ranges_;              // every range of every upstream block, by address
  std::set<std::pair<size_t, char*>> free_;    // the free ones, by size then address (best fit)
  std::vector<std::pair<void*, size_t>> upstream_;
  size_t reserved_ = 0;
  size_t live_     = 0;
  size_t maximum_  = 0;
  bool managed_    = false;
  int device_      = 0;
};

std::shared_ptr<pool> make_pool(size_t initial_bytes, size_t maximum_bytes, bool managed)
{
  return std::make_shared<pool>(initial_bytes, maximum_bytes, managed);
}
void* pool_allocate(pool& p, size_t bytes, hipStream_t stream, bool ordered)
{
  return p.allocate(bytes, stream, ordered);
}
bool pool_deallocate(pool& p, void* ptr, hipStream_t stream, bool ordered)
{
  return p.deallocate(ptr, stream, ordered);
}
size_t pool_reserved_bytes(const pool& p) { return p.reserved_bytes(); }
size_t pool_live_allocations(const pool& p) { return p.live_allocations(); }

namespace {
enum class source { plain, pooled, async };

/** Never destroyed: objects that outlive main() (a Python interpreter's indexes) still release
 *  their memory through it. */
struct process_state {
  std::mutex mutex;
  source how = source::plain;
  std::shared_ptr<pool> current;
  std::vector<std::shared_ptr<pool>> retired;  // switched away from while ranges were still live
  std::unordered_set<void*> async_live;        // addresses handed out by hipMallocAsync
};

process_state& state()
{
  static process_state* s = new process_state;
  return *s;
}

/** The pool that owns `ptr`, current or retired. */
std::shared_ptr<pool> owner_of(process_state& s, const void* ptr)
{
  if (s.current && s.current->owns(ptr)) { return s.current; }
  for (auto& p : s.retired) {
    if (p->owns(ptr)) { return p; }
  }
  return nullptr;
}

void drop_empty_retired(process_state& s)
{
  s.retired.erase(std::remove_if(s.retired.begin(), s.retired.end(),
                                 [](const std::shared_ptr<pool>& p) { return p->live_allocations() == 0; }),
                  s.retired.end());
}

void switch_to(source how, std::shared_ptr<pool> next)
{
  process_state& s = state();
  std::shared_ptr<pool> old;
  {
    std::lock_guard<std::mutex> lock(s.mutex);
    old       = std::move(s.current);
    s.current = std::move(next);
    s.how     = how;
    if (old && old->live_allocations() > 0) { s.retired.push_back(old); }
    drop_empty_retired(s);
  }
  // `old` (when nothing is live in it) returns its blocks to the device here, outside the lock
}
}  // namespace

size_t percent_of_free_device_memory(int percent)
{
  CUVS_EXPECTS(percent >= 0 && percent <= 100, "a percentage of the free memory must be within [0, 100]");
  size_t free_b = 0, total_b = 0;
  CUVS_HIP_TRY(hipMemGetInfo(&free_b, &total_b));
  return size_t(double(free_b) * double(percent) / 100.0) / kGranule * kGranule;
}

void* allocate(size_t bytes)
{
  process_state& s = state();
  std::shared_ptr<pool> p;
  {
    std::lock_guard<std::mutex> lock(s.mutex);
    if (s.how == source::pooled) { p = s.current; }
  }
  if (p) { return p->allocate(bytes, nullptr, false); }
  void* ptr = nullptr;
  CUVS_HIP_TRY(hipMalloc(&ptr, bytes));
  note_allocated(ptr, bytes);
  return ptr;
}

void deallocate(void* ptr) noexcept
{
  if (ptr == nullptr) { return; }
  process_state& s = state();
  std::shared_ptr<pool> p;
  {
    std::lock_guard<std::mutex> lock(s.mutex);
    p = owner_of(s, ptr);
    if (!p) { s.async_live.erase(ptr); }
  }
  if (p) {
    try {
      p->deallocate(ptr, nullptr, false);
    } catch (...) {
    }
    std::lock_guard<std::mutex> lock(s.mutex);
    drop_empty_retired(s);
    return;
  }
  note_released(ptr);
  (void)hipFree(ptr);  // also releases what hipMallocAsync handed out, after waiting for the device
}

void* allocate_on_stream(size_t bytes, hipStream_t stream)
{
  process_state& s = state();
  std::shared_ptr<pool> p;
  source how;
  {
    std::lock_guard<std::mutex> lock(s.mutex);
    how = s.how;
    p   = s.current;
  }
  if (how == source::pooled && p) { return p->allocate(bytes, stream, true); }
  void* ptr = nullptr;
  if (how == source::async) {
    CUVS_HIP_TRY(hipMallocAsync(&ptr, bytes == 0 ? 1 : bytes, stream));
    note_allocated(ptr, bytes);
    std::lock_guard<std::mutex> lock(s.mutex);
    s.async_live.insert(ptr);
    return ptr;
  }
  CUVS_HIP_TRY(hipMalloc(&ptr, bytes));
  note_allocated(ptr, bytes);
  return ptr;
}

void deallocate_on_stream(void* ptr, hipStream_t stream)
{
  if (ptr == nullptr) { return; }
  process_state& s = state();
  std::shared_ptr<pool> p;
  bool from_async = false;
  {
    std::lock_guard<std::mutex> lock(s.mutex);
    p = owner_of(s, ptr);
    if (!p) { from_async = s.async_live.erase(ptr) > 0; }
  }
  if (p) {
    p->deallocate(ptr, stream, true);
    std::lock_guard<std::mutex> lock(s.mutex);
    drop_empty_retired(s);
    return;
  }
  note_released(ptr);
  if (from_async) {
    CUVS_HIP_TRY(hipFreeAsync(ptr, stream));
    return;
  }
  CUVS_HIP_TRY(hipFree(ptr));
}

void* host_allocate(size_t bytes)
{
  void* ptr = nullptr;
  CUVS_HIP_TRY(hipHostMalloc(&ptr, bytes == 0 ? 1 : bytes, hipHostMallocDefault));
  note_allocated(ptr, bytes, space::pinned);
  return ptr;
}

void host_deallocate(void* ptr)
{
  if (ptr == nullptr) { return; }
  note_released(ptr);
  CUVS_HIP_TRY(hipHostFree(ptr));
}

void enable_pool(int initial_percent, int maximum_percent, bool managed)
{
  const size_t initial = percent_of_free_device_memory(initial_percent);
  const size_t maximum = percent_of_free_device_memory(maximum_percent);
  CUVS_EXPECTS(maximum > 0, "the maximum pool size must be more than 0 percent of the free memory");
  switch_to(source::pooled, make_pool(initial, maximum, managed));
}

void enable_async()
{
  int device = 0, supported = 0;
  CUVS_HIP_TRY(hipGetDevice(&device));
  CUVS_HIP_TRY(hipDeviceGetAttribute(&supported, hipDeviceAttributeMemoryPoolsSupported, device));
  CUVS_EXPECTS(supported != 0, "this device has no stream-ordered memory allocator");
  switch_to(source::async, nullptr);
}

void reset() { switch_to(source::plain, nullptr); }

}  // namespace cuvs::memory
