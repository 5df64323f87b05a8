/*
 * A plain C99 caller of the C ABI, the way a user of cuVS's C API would write it
 * (the flow of the reference's c/tests/neighbors/run_ivf_pq_c.c: create resources, build, search):
 * build an index from device memory, search it, save it, load it into a second index, search again.
 * Exits 0 when every call succeeds, the results are well formed, the rows find themselves, the
 * reloaded index answers identically and a wrong call reports an error with a message.
 *
 *   gcc -std=c99 -D__HIP_PLATFORM_AMD__ -Iinclude -I/opt/rocm/include tests/c_abi/ivf_pq_roundtrip.c \
 *       -Lcuvs_amd -lcuvs_c -L/opt/rocm/lib -lamdhip64 -Wl,-rpath,$PWD/cuvs_amd -o /tmp/ivf_pq_roundtrip
 */
#include <cuvs/core/c_api.h>
#include <cuvs/neighbors/ivf_pq.h>

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define N_ROWS 20000
#define DIM 32
#define N_QUERIES 200
#define K 10

#define CHECK(call)                                                                          \
  do {                                                                                       \
    if ((call) != CUVS_SUCCESS) {                                                            \
      const char* text = cuvsGetLastErrorText();                                             \
      fprintf(stderr, "%s:%d: %s failed: %s\n", __FILE__, __LINE__, #call, text ? text : ""); \
      return 1;                                                                              \
    }                                                                                        \
  } while (0)

static uint32_t lcg(uint32_t* s)
{
  *s = *s * 1664525u + 1013904223u;
  return *s >> 8;
}

static DLManagedTensor matrix(void* data, int64_t* shape, uint8_t code, uint8_t bits)
{
  DLManagedTensor t;
  memset(&t, 0, sizeof(t));
  t.dl_tensor.data               = data;
  t.dl_tensor.device.device_type = kDLROCM;
  t.dl_tensor.ndim               = 2;
  t.dl_tensor.dtype.code         = code;
  t.dl_tensor.dtype.bits         = bits;
  t.dl_tensor.dtype.lanes        = 1;
  t.dl_tensor.shape              = shape;
  return t;
}

static char last_search_error[512]; /* message of the last failed cuvsIvfPqSearch (later calls that succeed clear it) */

static int search(cuvsResources_t res, cuvsIvfPqIndex_t index, void* d_queries, int64_t n_queries,
                  int64_t dim, int64_t* h_neighbors, float* h_distances)
{
  void *d_neighbors = NULL, *d_distances = NULL;
  CHECK(cuvsRMMAlloc(res, &d_neighbors, sizeof(int64_t) * n_queries * K));
  CHECK(cuvsRMMAlloc(res, &d_distances, sizeof(float) * n_queries * K));
  int64_t q_shape[2] = {n_queries, dim}, o_shape[2] = {n_queries, K};
  DLManagedTensor queries   = matrix(d_queries, q_shape, kDLFloat, 32);
  DLManagedTensor neighbors = matrix(d_neighbors, o_shape, kDLInt, 64);
  DLManagedTensor distances = matrix(d_distances, o_shape, kDLFloat, 32);
  cuvsIvfPqSearchParams_t sp;
  CHECK(cuvsIvfPqSearchParamsCreate(&sp));
  sp->n_probes = 16;
  const cuvsError_t rc = cuvsIvfPqSearch(res, sp, index, &queries, &neighbors, &distances);
  last_search_error[0] = 0;
  if (rc != CUVS_SUCCESS && cuvsGetLastErrorText() != NULL) {
    strncpy(last_search_error, cuvsGetLastErrorText(), sizeof(last_search_error) - 1);
  }
  if (rc == CUVS_SUCCESS) {
    CHECK(cuvsStreamSync(res));
    if (hipMemcpy(h_neighbors, d_neighbors, sizeof(int64_t) * n_queries * K, hipMemcpyDeviceToHost) != hipSuccess ||
        hipMemcpy(h_distances, d_distances, sizeof(float) * n_queries * K, hipMemcpyDeviceToHost) != hipSuccess) {
      return 1;
    }
  }
  CHECK(cuvsIvfPqSearchParamsDestroy(sp));
  CHECK(cuvsRMMFree(res, d_neighbors, sizeof(int64_t) * n_queries * K));
  CHECK(cuvsRMMFree(res, d_distances, sizeof(float) * n_queries * K));
  return rc == CUVS_SUCCESS ? 0 : 2;
}

int main(int argc, char** argv)
{
  const char* path = argc > 1 ? argv[1] : "/tmp/ivf_pq_roundtrip.index";
  cuvsResources_t res;
  CHECK(cuvsResourcesCreate(&res));

  /* 40 clusters of rows around random centres */
  float* h_data = (float*)malloc(sizeof(float) * N_ROWS * DIM);
  float centres[40][DIM];
  uint32_t seed = 12345u;
  for (int c = 0; c < 40; c++) {
    for (int d = 0; d < DIM; d++) { centres[c][d] = (float)(lcg(&seed) % 2000) / 100.0f; }
  }
  for (int i = 0; i < N_ROWS; i++) {
    const int c = (int)(lcg(&seed) % 40);
    for (int d = 0; d < DIM; d++) { h_data[i * DIM + d] = centres[c][d] + (float)(lcg(&seed) % 1000) / 500.0f; }
  }
  void* d_data = NULL;
  CHECK(cuvsRMMAlloc(res, &d_data, sizeof(float) * N_ROWS * DIM));
  if (hipMemcpy(d_data, h_data, sizeof(float) * N_ROWS * DIM, hipMemcpyHostToDevice) != hipSuccess) { return 1; }

  int64_t shape[2]        = {N_ROWS, DIM};
  DLManagedTensor dataset = matrix(d_data, shape, kDLFloat, 32);
  cuvsIvfPqIndexParams_t ip;
  CHECK(cuvsIvfPqIndexParamsCreate(&ip));
  ip->n_lists = 64;
  ip->pq_dim  = 16;
  cuvsIvfPqIndex_t index;
  CHECK(cuvsIvfPqIndexCreate(&index));
  CHECK(cuvsIvfPqBuild(res, ip, &dataset, index));
  int64_t size = 0, n_lists = 0;
  CHECK(cuvsIvfPqIndexGetSize(index, &size));
  CHECK(cuvsIvfPqIndexGetNLists(index, &n_lists));
  if (size != N_ROWS || n_lists != 64) { fprintf(stderr, "size %ld lists %ld\n", (long)size, (long)n_lists); return 1; }

  /* the first rows as queries: each finds itself, distances ascend, ids are rows */
  static int64_t nb[N_QUERIES * K], nb2[N_QUERIES * K];
  static float dist[N_QUERIES * K], dist2[N_QUERIES * K];
  if (search(res, index, d_data, N_QUERIES, DIM, nb, dist) != 0) { return 1; }
  int self = 0;
  for (int q = 0; q < N_QUERIES; q++) {
    self += nb[q * K] == q;
    for (int r = 0; r < K; r++) {
      if (nb[q * K + r] < 0 || nb[q * K + r] >= N_ROWS) { fprintf(stderr, "id out of range\n"); return 1; }
      if (r > 0 && dist[q * K + r] < dist[q * K + r - 1]) { fprintf(stderr, "distances not ascending\n"); return 1; }
    }
  }
  if (self < N_QUERIES * 9 / 10) { fprintf(stderr, "only %d of %d rows found themselves\n", self, N_QUERIES); return 1; }

  /* save, load into a second index, same answers */
  CHECK(cuvsIvfPqSerialize(res, path, index));
  cuvsIvfPqIndex_t loaded;
  CHECK(cuvsIvfPqIndexCreate(&loaded));
  CHECK(cuvsIvfPqDeserialize(res, path, loaded));
  if (search(res, loaded, d_data, N_QUERIES, DIM, nb2, dist2) != 0) { return 1; }
  if (memcmp(nb, nb2, sizeof(nb)) != 0 || memcmp(dist, dist2, sizeof(dist)) != 0) {
    fprintf(stderr, "the reloaded index answers differently\n");
    return 1;
  }

  /* a wrong call: queries of another dimension -> CUVS_ERROR and a message, no crash */
  if (search(res, index, d_data, N_QUERIES, DIM / 2, nb2, dist2) != 2 || last_search_error[0] == 0) {
    fprintf(stderr, "a dimension mismatch was not reported\n");
    return 1;
  }

  CHECK(cuvsIvfPqIndexDestroy(loaded));
  CHECK(cuvsIvfPqIndexDestroy(index));
  CHECK(cuvsIvfPqIndexParamsDestroy(ip));
  CHECK(cuvsRMMFree(res, d_data, sizeof(float) * N_ROWS * DIM));
  CHECK(cuvsResourcesDestroy(res));
  free(h_data);
  remove(path);
  printf("ok: %d of %d rows found themselves\n", self, N_QUERIES);
  return 0;
}
