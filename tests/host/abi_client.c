/* A host written in plain C against include/fairring_hip.h, with no PyTorch in
 * the process: allocates K device buffers with the HIP runtime, reduces them
 * through the slice pipeline (frg_create / frg_allreduce / frg_work_wait) and
 * through one bare launch (frg_reduce_slice), and compares both with the same
 * left fold done on the host. Exit status 0 and the line "abi client ok" on
 * success. Usage: abi_client [K] [numel]                                      */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/fairring_hip.h"

#define CHECK_HIP(x)                                                      \
  do {                                                                    \
    hipError_t e_ = (x);                                                  \
    if (e_ != hipSuccess) {                                               \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));             \
      return 2;                                                           \
    }                                                                     \
  } while (0)

#define CHECK_FRG(x)                                                      \
  do {                                                                    \
    int rc_ = (x);                                                        \
    if (rc_ != FRG_OK) {                                                  \
      fprintf(stderr, "%s: status %d: %s\n", #x, rc_, frg_last_error());  \
      return 3;                                                           \
    }                                                                     \
  } while (0)

static uint32_t lcg(uint32_t* s) {
  *s = *s * 1664525u + 1013904223u;
  return *s;
}

int main(int argc, char** argv) {
  const int K = argc > 1 ? atoi(argv[1]) : 8;
  const int64_t n = argc > 2 ? atoll(argv[2]) : 1000003;
  if (K < 1 || K > 64 || n < 1) {
    fprintf(stderr, "usage: abi_client [K in 1..64] [numel]\n");
    return 1;
  }
  printf("abi %s, K = %d, numel = %lld\n", frg_version(), K, (long long)n);
  fflush(stdout);

  float** host = (float**)malloc(sizeof(float*) * (size_t)K);
  const void** dev = (const void**)malloc(sizeof(void*) * (size_t)K);
  float* want = (float*)malloc(sizeof(float) * (size_t)n);
  float* got = (float*)malloc(sizeof(float) * (size_t)n);
  uint32_t seed = 12345u;
  for (int k = 0; k < K; ++k) {
    host[k] = (float*)malloc(sizeof(float) * (size_t)n);
    for (int64_t i = 0; i < n; ++i) {
      host[k][i] = ((float)(lcg(&seed) >> 8) / 16777216.0f - 0.5f) * 0.02f;
    }
    void* d = NULL;
    CHECK_HIP(hipMalloc(&d, sizeof(float) * (size_t)n));
    CHECK_HIP(hipMemcpy(d, host[k], sizeof(float) * (size_t)n, hipMemcpyHostToDevice));
    dev[k] = d;
  }
  /* the contract: acc = x[0]; acc = acc + x[k] in index order; then * 1/K */
  const float scale = 1.0f / (float)K;
  for (int64_t i = 0; i < n; ++i) {
    volatile float acc = host[0][i];
    for (int k = 1; k < K; ++k) acc = acc + host[k][i];
    acc = acc * scale;
    want[i] = acc;
  }
  void* out = NULL;
  CHECK_HIP(hipMalloc(&out, sizeof(float) * (size_t)n));

  frg_options opts;
  memset(&opts, 0, sizeof(opts));
  opts.max_memory_allocated_in_bytes = 2 << 20;
  opts.slice_size_in_bytes = 1 << 20;
  frg_ctx* ctx = NULL;
  CHECK_FRG(frg_create(0, &opts, &ctx));
  frg_layout layout;
  CHECK_FRG(frg_get_layout(ctx, &layout));
  printf("layout: %lld slots of %lld bytes\n", (long long)layout.num_staging_slots,
         (long long)layout.slot_size_in_bytes);

  frg_work* work = NULL;
  CHECK_FRG(frg_allreduce(ctx, out, dev, K, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL, scale,
                          /*producer_stream=*/NULL, NULL, NULL, &work));
  CHECK_FRG(frg_work_wait(work));
  CHECK_FRG(frg_work_release(work));
  CHECK_HIP(hipMemcpy(got, out, sizeof(float) * (size_t)n, hipMemcpyDeviceToHost));
  if (memcmp(got, want, sizeof(float) * (size_t)n) != 0) {
    fprintf(stderr, "pipeline result differs from the host fold\n");
    return 4;
  }
  frg_progress progress;
  CHECK_FRG(frg_get_progress(ctx, &progress));
  printf("pipeline ok: %lld operation(s), %lld launches\n", (long long)progress.enqueued,
         (long long)progress.launches);

  CHECK_HIP(hipMemset(out, 0, sizeof(float) * (size_t)n));
  CHECK_FRG(frg_reduce_slice(out, dev, K, n, FRG_F32, FRG_SUM, FRG_SCALE_MUL, scale, 0, NULL));
  CHECK_HIP(hipDeviceSynchronize());
  CHECK_HIP(hipMemcpy(got, out, sizeof(float) * (size_t)n, hipMemcpyDeviceToHost));
  if (memcmp(got, want, sizeof(float) * (size_t)n) != 0) {
    fprintf(stderr, "single launch result differs from the host fold\n");
    return 5;
  }
  /* a contract violation comes back as a status and a message, not a crash */
  if (frg_reduce_slice(out, dev, 65, n, FRG_F32, FRG_SUM, FRG_SCALE_NONE, 1.0f, 0, NULL) !=
          FRG_ERR_INVALID ||
      strstr(frg_last_error(), "K must be") == NULL) {
    fprintf(stderr, "expected FRG_ERR_INVALID for K = 65\n");
    return 6;
  }
  CHECK_FRG(frg_destroy(ctx));
  printf("abi client ok\n");
  return 0;
}
