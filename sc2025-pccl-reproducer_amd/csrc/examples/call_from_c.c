/* The library called from plain C, the way the reference's own C++ would call it
 * in place of vectorAdd / ringReduceScatterGPU (pccl/src/reduce_scatter.cpp:127-152):
 * no torch, no Python.  Four virtual ranks on the current GPU, fp32:
 *   1. pccl_hip_accumulate        dst += src
 *   2. pccl_hip_reduce_scatter_virtual, "ring", per-step mode with caller-owned work buffers
 *   3. the same in the fused mode (no work buffers)
 *   4. pccl_hip_reduce_scatter_virtual_noalloc (work buffers built into the library)
 * Every result is compared bit for bit with the ring's left fold computed here on
 * the host.  Prints "OK" and returns 0, or says what differed.
 *
 * Build:  make -C sc2025-pccl-reproducer_amd/csrc example
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "pccl_hip.h"

#define P 4
#define B 100003 /* elements per block: not a multiple of the vector width */

#define HIP_OK(call)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)

#define PCCL_OK(call)                                                                  \
  do {                                                                                 \
    int rc_ = (call);                                                                  \
    if (rc_ != PCCL_HIP_OK) {                                                          \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, pccl_hip_last_error());      \
      return 3;                                                                        \
    }                                                                                  \
  } while (0)

static float pseudo(uint32_t* state) { /* uniform in [-1, 1) */
  *state = *state * 1664525u + 1013904223u;
  return (float)(*state >> 8) / 8388608.0f - 1.0f;
}

static int check(const char* what, void* const* d_out, float* const* want) {
  static float got[B];
  for (int r = 0; r < P; ++r) {
    HIP_OK(hipMemcpy(got, d_out[r], sizeof got, hipMemcpyDeviceToHost));
    if (memcmp(got, want[r], sizeof got) != 0) {
      fprintf(stderr, "%s: output of rank %d differs from the host fold\n", what, r);
      return 1;
    }
  }
  return 0;
}

int main(void) {
  static float h_in[P][P * B];
  float* want[P];
  void *d_in[P], *d_out[P], *d_work[P];
  uint32_t seed = 1234;

  if (pccl_hip_version() != PCCL_HIP_ABI_VERSION) {
    fprintf(stderr, "ABI version mismatch\n");
    return 4;
  }
  for (int r = 0; r < P; ++r)
    for (size_t i = 0; i < (size_t)P * B; ++i) h_in[r][i] = pseudo(&seed);

  /* block j lands on rank j: ((x[j+1] + x[j+2]) + ...) + x[j], ranks mod P */
  for (int j = 0; j < P; ++j) {
    want[j] = (float*)malloc(sizeof(float) * B);
    for (size_t i = 0; i < B; ++i) {
      volatile float acc = h_in[(j + 1) % P][(size_t)j * B + i];
      for (int t = 2; t <= P; ++t) acc = acc + h_in[(j + t) % P][(size_t)j * B + i];
      want[j][i] = acc;
    }
  }

  for (int r = 0; r < P; ++r) {
    HIP_OK(hipMalloc(&d_in[r], sizeof h_in[r]));
    HIP_OK(hipMalloc(&d_work[r], sizeof h_in[r]));
    HIP_OK(hipMalloc(&d_out[r], sizeof(float) * B));
    HIP_OK(hipMemcpy(d_in[r], h_in[r], sizeof h_in[r], hipMemcpyHostToDevice));
  }

  /* 1. accumulate: out0 = in0[0:B]; out0 += in1[0:B] */
  {
    static float got[B];
    HIP_OK(hipMemcpy(d_out[0], d_in[0], sizeof(float) * B, hipMemcpyDeviceToDevice));
    PCCL_OK(pccl_hip_accumulate(d_out[0], d_in[1], B, PCCL_HIP_F32, NULL));
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(got, d_out[0], sizeof got, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < B; ++i) {
      volatile float s = h_in[0][i] + h_in[1][i];
      if (memcmp(&got[i], (const void*)&s, 4) != 0) {
        fprintf(stderr, "accumulate: element %zu differs\n", i);
        return 1;
      }
    }
  }

  /* 2.-4. the ring reduce_scatter three ways */
  PCCL_OK(pccl_hip_reduce_scatter_virtual(d_out, (const void* const*)d_in, d_work, P, B, PCCL_HIP_F32, "ring",
                                          PCCL_HIP_MODE_STEPS, NULL));
  HIP_OK(hipDeviceSynchronize());
  if (check("per-step mode", d_out, want)) return 1;

  for (int r = 0; r < P; ++r) HIP_OK(hipMemset(d_out[r], 0, sizeof(float) * B));
  PCCL_OK(pccl_hip_reduce_scatter_virtual(d_out, (const void* const*)d_in, NULL, P, B, PCCL_HIP_F32, "ring",
                                          PCCL_HIP_MODE_FUSED, NULL));
  HIP_OK(hipDeviceSynchronize());
  if (check("fused mode", d_out, want)) return 1;

  for (int r = 0; r < P; ++r) HIP_OK(hipMemset(d_out[r], 0, sizeof(float) * B));
  PCCL_OK(pccl_hip_reduce_scatter_virtual_noalloc(d_out, (const void* const*)d_in, P, B, PCCL_HIP_F32, "ring", NULL));
  HIP_OK(hipDeviceSynchronize());
  if (check("built-in work buffers", d_out, want)) return 1;

  /* an argument error is a code and a message, never an exit */
  if (pccl_hip_reduce_scatter_virtual(d_out, (const void* const*)d_in, d_work, P, B, PCCL_HIP_F32, "tree",
                                      PCCL_HIP_MODE_STEPS, NULL) != PCCL_HIP_EINVAL ||
      strstr(pccl_hip_last_error(), "Unknown algorithm") == NULL) {
    fprintf(stderr, "unknown algorithm was not refused as documented\n");
    return 1;
  }

  for (int r = 0; r < P; ++r) {
    hipFree(d_in[r]); hipFree(d_work[r]); hipFree(d_out[r]); free(want[r]);
  }
  printf("OK\n");
  return 0;
}
