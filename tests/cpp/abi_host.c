/* A host written in C that uses the library through include/tandem_hip.h and nothing else of this
 * repository: no Python, no torch. Four rank buffers from hipMalloc, integer-valued fp32 data (so that
 * every sum and every division by four is exact and the expected bits need no oracle), then the ring
 * collectives of buffer ranks in both of their forms, the single-launch all-reduce, one AdamW step
 * with zero gradients and no decay (which must leave the parameters alone), and the refusals that a
 * C caller sees as status codes. Exit status 0 and "abi_host: ok" when everything matched.
 * Built by __graft_entry__.build() with gcc; run on the GPU by tests/test_gpu_c_host.py. */

#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/tandem_hip.h"

#define WORLD 4
#define N 100003 /* odd: the chunks start off the 16-byte grid */

#define HIP_OK(call)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)

#define TDM_OK_(call)                                                                  \
  do {                                                                                 \
    int s_ = (call);                                                                   \
    if (s_ != TDM_OK) {                                                                \
      fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, s_, tdm_last_error()); \
      return 3;                                                                        \
    }                                                                                  \
  } while (0)

static float host_in[WORLD][N], host_out[WORLD][N];
static void* dev[WORLD];

static float value(int rank, int i) { return (float)(((i * 7 + rank * 13) % 201) - 100) * 4.0f; } /* multiples of 4 */

static int upload(void) {
  for (int r = 0; r < WORLD; ++r) HIP_OK(hipMemcpy(dev[r], host_in[r], sizeof host_in[r], hipMemcpyHostToDevice));
  return 0;
}

static int download(void) {
  HIP_OK(hipDeviceSynchronize());
  for (int r = 0; r < WORLD; ++r) HIP_OK(hipMemcpy(host_out[r], dev[r], sizeof host_out[r], hipMemcpyDeviceToHost));
  return 0;
}

static int all_equal_the_mean(const char* what) {
  for (int r = 0; r < WORLD; ++r)
    for (int i = 0; i < N; ++i) {
      const float want = (host_in[0][i] + host_in[1][i] + host_in[2][i] + host_in[3][i]) / 4.0f;
      if (memcmp(&host_out[r][i], &want, 4) != 0) {
        fprintf(stderr, "%s: rank %d element %d is %g, expected %g\n", what, r, i, host_out[r][i], want);
        return 1;
      }
    }
  return 0;
}

int main(void) {
  int count = 0;
  HIP_OK(hipGetDeviceCount(&count));
  if (count < 1) {
    fprintf(stderr, "abi_host: no GPU\n");
    return 2;
  }
  HIP_OK(hipSetDevice(0));
  if (tdm_abi_version() < 1) return 3;
  for (int r = 0; r < WORLD; ++r) {
    HIP_OK(hipMalloc(&dev[r], sizeof host_in[r]));
    for (int i = 0; i < N; ++i) host_in[r][i] = value(r, i);
  }
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  /* the ring as W-1 launches per collective, then as one launch each, then the single-launch all-reduce */
  for (int form = 0; form <= 1; ++form) {
    TDM_OK_(tdm_set_ring_form(form));
    if (upload()) return 2;
    TDM_OK_(tdm_local_all_reduce(dev, WORLD, N, TDM_F32, 1, TDM_ALLREDUCE_RING, stream));
    if (download() || all_equal_the_mean(form ? "ring all-reduce, one launch per collective" : "ring all-reduce, steps")) return 1;
    /* reduce-scatter then all-gather as two calls, with explicit chunk sizes, one of them empty */
    const int64_t sizes[WORLD] = {N - 7000, 0, 6999, 1};
    if (upload()) return 2;
    TDM_OK_(tdm_local_reduce_scatter(dev, WORLD, N, TDM_F32, sizes, WORLD, 1, 1, stream));
    TDM_OK_(tdm_local_all_gather(dev, WORLD, N, TDM_F32, sizes, WORLD, stream));
    if (download() || all_equal_the_mean("reduce-scatter + all-gather")) return 1;
  }
  TDM_OK_(tdm_set_ring_form(-1));
  if (upload()) return 2;
  TDM_OK_(tdm_local_all_reduce(dev, WORLD, N, TDM_F32, 1, TDM_ALLREDUCE_FOLD, stream));
  if (download() || all_equal_the_mean("single-launch all-reduce")) return 1;

  /* what a C caller gets for bad arguments: a status and a message, nothing launched */
  if (tdm_local_all_reduce(dev, WORLD, N, 42, 0, TDM_ALLREDUCE_RING, stream) != TDM_EINVAL || strstr(tdm_last_error(), "dtype") == NULL) {
    fprintf(stderr, "an unknown dtype was not refused: %s\n", tdm_last_error());
    return 1;
  }
  if (tdm_local_all_reduce(dev, WORLD, N, TDM_I32, 1, TDM_ALLREDUCE_RING, stream) != TDM_EINVAL) {
    fprintf(stderr, "averaging integers was not refused\n");
    return 1;
  }
  void* aliased[WORLD] = {dev[0], dev[0], dev[2], dev[3]};
  if (tdm_local_all_reduce(aliased, WORLD, N, TDM_F32, 0, TDM_ALLREDUCE_RING, stream) != TDM_EINVAL) {
    fprintf(stderr, "two ranks sharing a buffer were not refused\n");
    return 1;
  }
  char name[128];
  int cus = 0;
  int64_t bytes = 0;
  TDM_OK_(tdm_device_info(0, name, sizeof name, &cus, &bytes));
  HIP_OK(hipStreamDestroy(stream));
  for (int r = 0; r < WORLD; ++r) HIP_OK(hipFree(dev[r]));
  printf("abi_host: ok (%s, %d compute units)\n", name, cus);
  return 0;
}
