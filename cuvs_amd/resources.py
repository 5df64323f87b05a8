"""Mirror of cuvs.common.Resources (python/cuvs/cuvs/common/resources.pyx): owns a cuvsResources_t."""
import ctypes as C

from ._lib import SearchTuningStruct, check, lib


class Resources:
    def __init__(self, stream=None, memory_tracking_csv_path=None, memory_tracking_sample_interval_ms=10):
        """`memory_tracking_csv_path`: the handle also counts the library's allocations and writes samples
        to that CSV file until it is destroyed (resources.pyx:75-84)."""
        self._h = C.c_size_t(0)
        if memory_tracking_csv_path:
            check(lib().cuvsResourcesCreateWithMemoryTracking(
                C.byref(self._h), str(memory_tracking_csv_path).encode("utf-8"),
                int(memory_tracking_sample_interval_ms)))
        else:
            check(lib().cuvsResourcesCreate(C.byref(self._h)))
        if stream is not None:
            self.set_stream(stream)

    def set_stream(self, stream):
        """`stream` is a raw hipStream_t value or an object with a `cuda_stream` attribute."""
        raw = getattr(stream, "cuda_stream", stream)
        check(lib().cuvsStreamSet(self._h, C.c_void_p(raw)))

    def use_torch_current_stream(self):
        import torch
        self.set_stream(torch.cuda.current_stream().cuda_stream)

    def sync(self):
        check(lib().cuvsStreamSync(self._h))

    def set_workspace_pool(self, initial_size_bytes):
        """Give the handle a device memory pool of its own (cuvsResourcesSetWorkspacePool): the search
        workspace then comes out of memory reserved here instead of a device allocation on first use."""
        check(lib().cuvsResourcesSetWorkspacePool(self._h, C.c_size_t(int(initial_size_bytes))))

    def get_c_obj(self):
        return self._h

    def set_search_tuning(self, early_stop="auto", generic_scan=False, plain_coarse=False, serial_batches=False):
        """cuvsAmdIvfPqSetSearchTuning: fix choices the search otherwise makes by itself (results do
        not depend on them).  early_stop: "auto", "off" (every probed list streamed in full) or "on";
        serial_batches: internal batches one after the other instead of side by side."""
        t = SearchTuningStruct()
        t.early_stop = {"auto": 0, "off": 1, "on": 2}[early_stop]
        t.generic_scan = int(bool(generic_scan))
        t.plain_coarse = int(bool(plain_coarse))
        t.serial_batches = int(bool(serial_batches))
        check(lib().cuvsAmdIvfPqSetSearchTuning(self._h, C.byref(t)))

    def enable_profiling(self, on=True):
        check(lib().cuvsAmdIvfPqProfilingEnable(self._h, bool(on)))

    def __del__(self):
        try:
            if self._h.value:
                lib().cuvsResourcesDestroy(self._h)
                self._h = C.c_size_t(0)
        except Exception:
            pass


def pool_memory_resource_enable(initial_pool_size_percent, max_pool_size_percent, managed=False):
    """One device memory pool for the whole process (cuvsRMMPoolMemoryResourceEnable; the Go binding's
    memory_resource.go:58 makes the same call)."""
    check(lib().cuvsRMMPoolMemoryResourceEnable(int(initial_pool_size_percent), int(max_pool_size_percent),
                                                bool(managed)))


def async_memory_resource_enable():
    check(lib().cuvsRMMAsyncMemoryResourceEnable())


def memory_resource_reset():
    check(lib().cuvsRMMMemoryResourceReset())
