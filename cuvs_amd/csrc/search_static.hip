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
 * Consequences of the one array per GPU: calls that overlap on one GPU (from several host threads
 * or on several streams) race on it; the array keeps the previous call's contents, and the
 * search initialises every counter, bound and flag it reads (as it must on the cached workspace,
 * which is reused the same way).
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
    local.set_stream(caller->stream());
    local.borrow_workspace(static_scratch(), kStaticScratchBytes);
    cuvs::core::ivf_pq_search_tensors(local, search_params, index, queries, neighbors, distances,
                                      nullptr, 0);
  });
}
