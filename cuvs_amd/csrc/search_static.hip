/*
 * cuvsAmdIvfPqSearchNoAlloc: cuvsIvfPqSearch for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 *
 * The search keeps everything between its stages in a per-call workspace: mapped and rotated
 * queries, coarse scores, probes, chunk indices, the pair records in list order, survivor lists
 * and counters of the early stop, and the candidate keys every (query, probe) pair hands to the
 * per-query merge.  cuvsIvfPqSearch takes that workspace from the handle's cached allocation,
 * which grows on demand.  Here it is a fixed array in device memory that is part of the library's
 * code object: every GPU the library is loaded on holds its own copy from load to process exit.
 * The kernels are the ones cuvsIvfPqSearch launches and get their buffers as arguments as there.
 *
 * Consequences of the one array per GPU: calls on different streams of one GPU take turns (each
 * waits for an event recorded behind the call before it), but calls issued from several host
 * threads at once, and captured calls replayed side by side, race on it; the array keeps the
 * previous call's contents, and the search initialises every counter, bound and flag it reads (as
 * it must on the cached workspace, which is reused the same way).  A call larger than the array
 * runs in internal batches that fit; only a single query that does not fit is refused.
 */
#include <hip/hip_runtime.h>

#include "c_common.hpp"

#include <mutex>

namespace {

constexpr size_t kStaticScratchBytes = CUVS_AMD_NO_ALLOC_WORKSPACE_BYTES;
constexpr int kMaxDevices            = 64;

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices] = {};
// recorded behind every call on a device: the next call's stream waits for it, so that calls on
// different streams or handles take turns on the one array (not under stream capture: a captured
// call is ordered by its graph's launches, and two graphs that hold such calls must not overlap)
hipEvent_t scratch_free[kMaxDevices] = {};

/** Device address of the current device's copy of `scratch` (looked up once per device). */
void* static_scratch()
{
  int device = 0;
  CUVS_HIP_TRY(hipGetDevice(&device));
  CUVS_EXPECTS(device >= 0 && device < kMaxDevices, "device ordinal %d is out of range", device);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[device] == nullptr) {
    void* p = nullptr;
    CUVS_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    CUVS_EXPECTS(p != nullptr && reinterpret_cast<uintptr_t>(p) % 256 == 0,
                 "the static workspace has no usable device address");
    scratch_ptr[device] = p;
  }
  return scratch_ptr[device];
}

}  // namespace

extern "C" cuvsError_t cuvsAmdIvfPqSearchNoAlloc(cuvsResources_t res,
                                                 cuvsIvfPqSearchParams_t search_params,
                                                 cuvsIvfPqIndex_t index,
                                                 DLManagedTensor* queries,
                                                 DLManagedTensor* neighbors,
                                                 DLManagedTensor* distances)
{
  return cuvs::core::translate_exceptions([=] {
    cuvs::resources* caller = cuvs::core::res_of(res);
    // a handle of this call's own: the caller's stream, the static array as the whole workspace
    cuvs::resources local;
    hipStream_t stream = caller->stream();
    local.set_stream(stream);
    local.tuning = caller->tuning;
    local.borrow_workspace(static_scratch(), kStaticScratchBytes);
    int device = 0;
    CUVS_HIP_TRY(hipGetDevice(&device));
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    CUVS_HIP_TRY(hipStreamIsCapturing(stream, &capture));
    hipEvent_t turn = nullptr;
    if (capture == hipStreamCaptureStatusNone) {
      std::lock_guard<std::mutex> lock(scratch_mutex);
      if (scratch_free[device] == nullptr) {
        CUVS_HIP_TRY(hipEventCreateWithFlags(&scratch_free[device], hipEventDisableTiming));
      } else {
        CUVS_HIP_TRY(hipStreamWaitEvent(stream, scratch_free[device], 0));
      }
      turn = scratch_free[device];
    }
    cuvs::core::ivf_pq_search_tensors(local, search_params, index, queries, neighbors, distances,
                                      nullptr, 0);
    if (turn != nullptr) {
      std::lock_guard<std::mutex> lock(scratch_mutex);
      CUVS_HIP_TRY(hipEventRecord(turn, stream));
    }
  });
}
