/*
 * C99 caller of the core C ABI: resources, the three device memory sources, pinned host memory,
 * matrix copies and row slices.  The sequence of calls follows the reference's own test of these
 * entry points (c/tests/core/c_api.c); the checks of what comes back are added here.
 */
#include <cuvs/core/c_api.h>
#include <cuvs/version_config.h>

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define CHECK(cond)                                                                  \
  do {                                                                               \
    if (!(cond)) {                                                                   \
      const char* text_ = cuvsGetLastErrorText();                                    \
      printf("FAILED %s:%d: %s (%s)\n", __FILE__, __LINE__, #cond, text_ ? text_ : "no error text"); \
      exit(EXIT_FAILURE);                                                            \
    }                                                                                \
  } while (0)

static void fill_and_check(cuvsResources_t res, hipStream_t stream, void* dev, size_t bytes, int value)
{
  unsigned char* host = (unsigned char*)malloc(bytes);
  CHECK(hipMemsetAsync(dev, value, bytes, stream) == hipSuccess);
  CHECK(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, stream) == hipSuccess);
  CHECK(cuvsStreamSync(res) == CUVS_SUCCESS);
  for (size_t i = 0; i < bytes; i++) { CHECK(host[i] == (unsigned char)value); }
  free(host);
}

static DLManagedTensor matrix(void* data, int64_t* shape, int64_t* strides, DLDeviceType where)
{
  DLManagedTensor t;
  memset(&t, 0, sizeof(t));
  t.dl_tensor.data               = data;
  t.dl_tensor.device.device_type = where;
  t.dl_tensor.ndim               = 2;
  t.dl_tensor.dtype.code         = kDLFloat;
  t.dl_tensor.dtype.bits         = 32;
  t.dl_tensor.dtype.lanes        = 1;
  t.dl_tensor.shape              = shape;
  t.dl_tensor.strides            = strides;
  return t;
}

int main(void)
{
  cuvsResources_t res;
  CHECK(cuvsResourcesCreate(&res) == CUVS_SUCCESS);
  hipStream_t stream;
  CHECK(hipStreamCreate(&stream) == hipSuccess);
  CHECK(cuvsStreamSet(res, stream) == CUVS_SUCCESS);

  /* plain device memory */
  void* ptr = NULL;
  CHECK(cuvsRMMAlloc(res, &ptr, 1024) == CUVS_SUCCESS && ptr != NULL);
  fill_and_check(res, stream, ptr, 1024, 0x11);
  CHECK(cuvsRMMFree(res, ptr, 1024) == CUVS_SUCCESS);

  /* one pool for the whole process: a freed range is handed out again, neighbours merge */
  CHECK(cuvsRMMPoolMemoryResourceEnable(1, 50, false) == CUVS_SUCCESS);
  void *a = NULL, *b = NULL, *c = NULL;
  CHECK(cuvsRMMAlloc(res, &a, 1024) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &b, 4096) == CUVS_SUCCESS);
  CHECK(a != NULL && b != NULL && a != b);
  CHECK((char*)b == (char*)a + 1024); /* carved back to back out of the reserved block */
  fill_and_check(res, stream, a, 1024, 0x22);
  fill_and_check(res, stream, b, 4096, 0x33);
  CHECK(cuvsRMMFree(res, a, 1024) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &c, 512) == CUVS_SUCCESS);
  CHECK(c == a); /* best fit: the 1024-byte hole, not the large remainder */
  CHECK(cuvsRMMFree(res, c, 512) == CUVS_SUCCESS);
  CHECK(cuvsRMMFree(res, b, 4096) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &c, 8192) == CUVS_SUCCESS);
  CHECK(c == a); /* everything merged back into one range */
  /* memory handed out by the pool outlives the switch back and is still released correctly */
  CHECK(cuvsRMMMemoryResourceReset() == CUVS_SUCCESS);
  fill_and_check(res, stream, c, 8192, 0x44);
  CHECK(cuvsRMMFree(res, c, 8192) == CUVS_SUCCESS);
  /* more than the maximum is refused with a message */
  CHECK(cuvsRMMPoolMemoryResourceEnable(0, 1, false) == CUVS_SUCCESS);
  size_t free_b = 0, total_b = 0;
  CHECK(hipMemGetInfo(&free_b, &total_b) == hipSuccess);
  CHECK(cuvsRMMAlloc(res, &ptr, free_b / 100 * 2) == CUVS_ERROR);
  CHECK(cuvsGetLastErrorText() != NULL && strstr(cuvsGetLastErrorText(), "pool exhausted") != NULL);
  CHECK(cuvsRMMMemoryResourceReset() == CUVS_SUCCESS);
  CHECK(cuvsRMMPoolMemoryResourceEnable(60, 50, false) == CUVS_ERROR);

  /* a pool over managed memory */
  CHECK(cuvsRMMPoolMemoryResourceEnable(0, 1, true) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &ptr, 1024) == CUVS_SUCCESS && ptr != NULL);
  fill_and_check(res, stream, ptr, 1024, 0x55);
  CHECK(cuvsRMMFree(res, ptr, 1024) == CUVS_SUCCESS);
  CHECK(cuvsRMMMemoryResourceReset() == CUVS_SUCCESS);

  /* the runtime's stream-ordered allocator */
  CHECK(cuvsRMMAsyncMemoryResourceEnable() == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &ptr, 1024) == CUVS_SUCCESS && ptr != NULL);
  fill_and_check(res, stream, ptr, 1024, 0x66);
  CHECK(cuvsRMMFree(res, ptr, 1024) == CUVS_SUCCESS);
  CHECK(cuvsRMMMemoryResourceReset() == CUVS_SUCCESS);

  /* a pool of the handle's own */
  CHECK(cuvsResourcesSetWorkspacePool(res, (size_t)64 << 20) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &a, 1 << 20) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &b, 1 << 20) == CUVS_SUCCESS);
  CHECK((char*)b == (char*)a + (1 << 20));
  CHECK(cuvsRMMFree(res, a, 1 << 20) == CUVS_SUCCESS);
  CHECK(cuvsRMMFree(res, b, 1 << 20) == CUVS_SUCCESS);
  CHECK(cuvsRMMAlloc(res, &c, (size_t)100 << 20) == CUVS_SUCCESS); /* grows past the reservation */
  fill_and_check(res, stream, c, 4096, 0x77);
  CHECK(cuvsRMMFree(res, c, (size_t)100 << 20) == CUVS_SUCCESS);

  /* pinned host memory */
  void* pinned = NULL;
  CHECK(cuvsRMMHostAlloc(&pinned, 1024) == CUVS_SUCCESS && pinned != NULL);
  memset(pinned, 0x5a, 1024);
  CHECK(cuvsRMMAlloc(res, &ptr, 1024) == CUVS_SUCCESS);
  CHECK(hipMemcpyAsync(ptr, pinned, 1024, hipMemcpyHostToDevice, stream) == hipSuccess);
  CHECK(cuvsStreamSync(res) == CUVS_SUCCESS);
  memset(pinned, 0, 1024);
  CHECK(hipMemcpyAsync(pinned, ptr, 1024, hipMemcpyDeviceToHost, stream) == hipSuccess);
  CHECK(cuvsStreamSync(res) == CUVS_SUCCESS);
  CHECK(((unsigned char*)pinned)[0] == 0x5a && ((unsigned char*)pinned)[1023] == 0x5a);
  CHECK(cuvsRMMFree(res, ptr, 1024) == CUVS_SUCCESS);
  CHECK(cuvsRMMHostFree(pinned, 1024) == CUVS_SUCCESS);

  /* matrix copy: host rows of 5 -> device rows padded to 8 -> host, and a slice of the rows */
  enum { ROWS = 7, COLS = 5, PAD = 8 };
  float host_in[ROWS * COLS], host_out[ROWS * COLS], host_slice[3 * COLS];
  for (int i = 0; i < ROWS * COLS; i++) { host_in[i] = (float)i * 0.5f; }
  void* dev = NULL;
  CHECK(cuvsRMMAlloc(res, &dev, ROWS * PAD * sizeof(float)) == CUVS_SUCCESS);
  int64_t shape[2] = {ROWS, COLS}, padded[2] = {PAD, 1};
  DLManagedTensor t_in  = matrix(host_in, shape, NULL, kDLCPU);
  DLManagedTensor t_dev = matrix(dev, shape, padded, kDLCUDA);
  DLManagedTensor t_out = matrix(host_out, shape, NULL, kDLCPU);
  CHECK(cuvsMatrixCopy(res, &t_in, &t_dev) == CUVS_SUCCESS);
  CHECK(cuvsMatrixCopy(res, &t_dev, &t_out) == CUVS_SUCCESS);
  CHECK(cuvsStreamSync(res) == CUVS_SUCCESS);
  CHECK(memcmp(host_in, host_out, sizeof(host_in)) == 0);
  DLManagedTensor view;
  memset(&view, 0, sizeof(view));
  CHECK(cuvsMatrixSliceRows(res, &t_dev, 2, 5, &view) == CUVS_SUCCESS);
  CHECK(view.dl_tensor.ndim == 2 && view.dl_tensor.shape[0] == 3 && view.dl_tensor.shape[1] == COLS);
  CHECK(view.dl_tensor.strides != NULL && view.dl_tensor.strides[0] == PAD);
  CHECK((char*)view.dl_tensor.data == (char*)dev + 2 * PAD * sizeof(float));
  int64_t slice_shape[2] = {3, COLS};
  DLManagedTensor t_slice = matrix(host_slice, slice_shape, NULL, kDLCPU);
  CHECK(cuvsMatrixCopy(res, &view, &t_slice) == CUVS_SUCCESS);
  CHECK(cuvsStreamSync(res) == CUVS_SUCCESS);
  CHECK(memcmp(host_slice, host_in + 2 * COLS, sizeof(host_slice)) == 0);
  view.deleter(&view);
  CHECK(view.dl_tensor.shape == NULL && view.dl_tensor.strides == NULL);
  /* what the copy refuses */
  int64_t other[2] = {ROWS, COLS + 1};
  DLManagedTensor t_bad = matrix(host_out, other, NULL, kDLCPU);
  CHECK(cuvsMatrixCopy(res, &t_in, &t_bad) == CUVS_ERROR);
  CHECK(strstr(cuvsGetLastErrorText(), "shape mismatch") != NULL);
  t_bad = matrix(host_out, shape, NULL, kDLCPU);
  t_bad.dl_tensor.dtype.bits = 16;
  CHECK(cuvsMatrixCopy(res, &t_in, &t_bad) == CUVS_ERROR);
  CHECK(cuvsMatrixSliceRows(res, &t_dev, 5, 2, &view) == CUVS_ERROR);
  CHECK(cuvsMatrixSliceRows(res, &t_dev, 0, ROWS + 1, &view) == CUVS_ERROR);
  CHECK(cuvsRMMFree(res, dev, ROWS * PAD * sizeof(float)) == CUVS_SUCCESS);

  CHECK(cuvsResourcesDestroy(res) == CUVS_SUCCESS);
  CHECK(hipStreamDestroy(stream) == hipSuccess);

  uint16_t major = 0, minor = 0, patch = 1;
  CHECK(cuvsVersionGet(&major, &minor, &patch) == CUVS_SUCCESS);
  CHECK(major == CUVS_VERSION_MAJOR && minor == CUVS_VERSION_MINOR && patch == CUVS_VERSION_PATCH);
  CHECK(major == 26 && minor == 10);
  printf("ok\n");
  return 0;
}
