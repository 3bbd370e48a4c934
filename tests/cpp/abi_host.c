/* A host written in C that uses the library through include/tandem_hip.h and nothing else of this
 * repository: no Python, no torch. Four rank buffers from hipMalloc, integer-valued fp32 data (so that
 * every sum and every division by four is exact and the expected bits need no oracle), then the ring
 * collectives of buffer ranks in both of their forms, the single-launch all-reduce, three AdamW steps
 * on a float64 shard through tdm_k3_adamw_typed (checked bit for bit against the same seven operations
 * written out in C doubles below), and the refusals that a C caller sees as status codes. Exit status 0 and "abi_host: ok" when everything matched.
 * Built by __graft_entry__.build() with gcc; run on the GPU by tests/test_gpu_c_host.py. */

#include <hip/hip_runtime_api.h>
#include <math.h>
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

/* tandem/optim.py:28-37 on doubles, operation for operation (lerp_ and addcmul_ fuse their last multiply-add). */
#define SHARD 4099
static double sp[SHARD], sg[SHARD], sm[SHARD], sv[SHARD], got_p[SHARD], got_m[SHARD], got_v[SHARD];

static int adamw_in_doubles(hipStream_t stream) {
  const double lr = 3e-4, beta1 = 0.9, beta2 = 0.95, eps = 1e-8, wd = 0.1;
  void *dp, *dg, *dm, *dv;
  HIP_OK(hipMalloc(&dp, sizeof sp));
  HIP_OK(hipMalloc(&dg, sizeof sg));
  HIP_OK(hipMalloc(&dm, sizeof sm));
  HIP_OK(hipMalloc(&dv, sizeof sv));
  for (int i = 0; i < SHARD; ++i) {
    sp[i] = 0.02 * sin(0.37 * i + 1.0);
    sm[i] = sv[i] = 0.0;
  }
  HIP_OK(hipMemcpy(dp, sp, sizeof sp, hipMemcpyHostToDevice));
  HIP_OK(hipMemset(dm, 0, sizeof sm));
  HIP_OK(hipMemset(dv, 0, sizeof sv));
  for (int step = 1; step <= 3; ++step) {
    for (int i = 0; i < SHARD; ++i) sg[i] = 1e-3 * cos(0.11 * i + step);
    HIP_OK(hipMemcpy(dg, sg, sizeof sg, hipMemcpyHostToDevice));
    tdm_adamw_hyper h;
    memset(&h, 0, sizeof h);
    h.use_decay = 1;
    h.decay = 1 - lr * wd;
    h.w1 = 1 - beta1;
    h.beta2 = beta2;
    h.one_m_b2 = 1 - beta2;
    h.bc2_sqrt = sqrt(1 - pow(beta2, step));
    h.eps = eps;
    h.neg_step = -(lr / (1 - pow(beta1, step)));
    TDM_OK_(tdm_k3_adamw_typed(dp, dg, dm, dv, SHARD, TDM_F64, &h, TDM_ADAMW_HOST_ORDER, NULL, 0, stream));
    for (int i = 0; i < SHARD; ++i) {
      sp[i] = sp[i] * h.decay;
      sm[i] = fma(h.w1, sg[i] - sm[i], sm[i]);
      sv[i] = fma(h.one_m_b2 * sg[i], sg[i], sv[i] * h.beta2);
      const double d = sqrt(sv[i]) / h.bc2_sqrt + h.eps;
      sp[i] = sp[i] + (h.neg_step * sm[i]) / d;
    }
  }
  HIP_OK(hipStreamSynchronize(stream));
  HIP_OK(hipMemcpy(got_p, dp, sizeof sp, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(got_m, dm, sizeof sm, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(got_v, dv, sizeof sv, hipMemcpyDeviceToHost));
  if (memcmp(got_p, sp, sizeof sp) || memcmp(got_m, sm, sizeof sm) || memcmp(got_v, sv, sizeof sv)) {
    fprintf(stderr, "AdamW on doubles: the GPU's bits differ from the same operations in C\n");
    return 1;
  }
  tdm_adamw_hyper h;
  memset(&h, 0, sizeof h);
  if (tdm_k3_adamw_typed(dp, dg, dm, dv, SHARD, TDM_I32, &h, TDM_ADAMW_HOST_ORDER, NULL, 0, stream) != TDM_EINVAL ||
      tdm_k3_adamw_typed(dp, dg, dm, dv, SHARD, TDM_F64, &h, TDM_ADAMW_DEVICE_ORDER, NULL, 0, stream) != TDM_EINVAL) {
    fprintf(stderr, "AdamW: an integer shard or the device order on doubles was not refused\n");
    return 1;
  }
  HIP_OK(hipFree(dp));
  HIP_OK(hipFree(dg));
  HIP_OK(hipFree(dm));
  HIP_OK(hipFree(dv));
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
  {
    const int status = adamw_in_doubles(stream);
    if (status) return status;
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
