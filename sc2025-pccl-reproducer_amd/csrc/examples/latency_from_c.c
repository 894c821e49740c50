/* What one call of the library costs for small messages, measured from plain C:
 * no Python, no ctypes, no torch.  bf16 messages of 4 KiB ... 1 MiB; per size
 * the microseconds per call (device time between two events around CALLS calls,
 * after WARM untimed ones) of
 *   accumulate          pccl_hip_accumulate                         (a1: pccl/src/common.cu:5-19)
 *   copy                pccl_hip_copy_batched, one segment
 *   rs_fused            pccl_hip_reduce_scatter_virtual, 8 ranks, "ring", one fused launch
 *   rs_steps            the same as 7 per-step launches
 *   rs_steps_graph      the 7 launches captured once into a HIP graph and replayed
 *   ag_fused            pccl_hip_all_gather_virtual, 8 ranks, one launch
 *   host_us_*           wall-clock microseconds the calling thread spends inside one call
 * Prints one JSON array.  Build:  make -C sc2025-pccl-reproducer_amd/csrc example
 */
#define __HIP_PLATFORM_AMD__ 1
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

#include "pccl_hip.h"

#define P 8
#define WARM 20
#define CALLS 200

#define HIP_OK(call)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess) {                                                            \
      fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                \
      exit(2);                                                                         \
    }                                                                                  \
  } while (0)

#define PCCL_OK(call)                                                                  \
  do {                                                                                 \
    int rc_ = (call);                                                                  \
    if (rc_ != PCCL_HIP_OK) {                                                          \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, pccl_hip_last_error());      \
      exit(3);                                                                         \
    }                                                                                  \
  } while (0)

static void *d_in[P], *d_out[P], *d_work[P], *d_gout[P], *d_x, *d_y, *d_z;
static size_t g_n, g_B;
static hipStream_t g_stream;
static hipGraphExec_t g_graph;

static void do_accumulate(void) { PCCL_OK(pccl_hip_accumulate(d_x, d_y, g_n, PCCL_HIP_BF16, g_stream)); }
static void do_copy(void) {
  void* dst[1] = {d_z};
  const void* src[1] = {d_x};
  size_t nb[1] = {g_n * 2};
  PCCL_OK(pccl_hip_copy_batched(dst, src, nb, 1, g_stream));
}
static void do_rs_fused(void) {
  PCCL_OK(pccl_hip_reduce_scatter_virtual(d_out, (const void* const*)d_in, NULL, P, g_B, PCCL_HIP_BF16, "ring",
                                          PCCL_HIP_MODE_FUSED, g_stream));
}
static void do_rs_steps(void) {
  PCCL_OK(pccl_hip_reduce_scatter_virtual(d_out, (const void* const*)d_in, d_work, P, g_B, PCCL_HIP_BF16, "ring",
                                          PCCL_HIP_MODE_STEPS, g_stream));
}
static void do_rs_graph(void) { HIP_OK(hipGraphLaunch(g_graph, g_stream)); }
static void do_ag_fused(void) {
  PCCL_OK(pccl_hip_all_gather_virtual(d_gout, (const void* const*)d_out, P, g_B * 2, "ring", PCCL_HIP_MODE_FUSED, g_stream));
}

static double now_us(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return t.tv_sec * 1e6 + t.tv_nsec * 1e-3;
}

/* device microseconds per call, and host microseconds spent inside a call */
static void measure(void (*fn)(void), double* dev_us, double* host_us) {
  hipEvent_t a, b;
  float ms;
  HIP_OK(hipEventCreate(&a));
  HIP_OK(hipEventCreate(&b));
  for (int i = 0; i < WARM; ++i) fn();
  HIP_OK(hipStreamSynchronize(g_stream));
  HIP_OK(hipEventRecord(a, g_stream));
  const double t0 = now_us();
  for (int i = 0; i < CALLS; ++i) fn();
  const double t1 = now_us();
  HIP_OK(hipEventRecord(b, g_stream));
  HIP_OK(hipStreamSynchronize(g_stream));
  HIP_OK(hipEventElapsedTime(&ms, a, b));
  *dev_us = ms * 1e3 / CALLS;
  *host_us = (t1 - t0) / CALLS;
  HIP_OK(hipEventDestroy(a));
  HIP_OK(hipEventDestroy(b));
}

int main(void) {
  const size_t max_bytes = 1 << 20;
  HIP_OK(hipStreamCreate(&g_stream));
  for (int r = 0; r < P; ++r) {
    HIP_OK(hipMalloc(&d_in[r], max_bytes));     /* P blocks of max_bytes / P */
    HIP_OK(hipMalloc(&d_work[r], max_bytes));
    HIP_OK(hipMalloc(&d_out[r], max_bytes / P));
    HIP_OK(hipMalloc(&d_gout[r], max_bytes));
    HIP_OK(hipMemset(d_in[r], 0, max_bytes));
  }
  HIP_OK(hipMalloc(&d_x, max_bytes));
  HIP_OK(hipMalloc(&d_y, max_bytes));
  HIP_OK(hipMalloc(&d_z, max_bytes));
  HIP_OK(hipMemset(d_x, 0, max_bytes));
  HIP_OK(hipMemset(d_y, 0, max_bytes));
  HIP_OK(hipDeviceSynchronize());

  printf("[");
  for (size_t bytes = 4096; bytes <= max_bytes; bytes *= 2) {
    double dev[6], host[6];
    hipGraph_t graph;
    g_n = bytes / 2;                 /* bf16 elements of the flat kernels */
    g_B = g_n / P;                   /* block of the 8-rank collectives: the message is one rank's input */
    do_rs_steps();                   /* loads the kernels before the capture */
    HIP_OK(hipStreamSynchronize(g_stream));
    HIP_OK(hipStreamBeginCapture(g_stream, hipStreamCaptureModeGlobal));
    do_rs_steps();
    HIP_OK(hipStreamEndCapture(g_stream, &graph));
    HIP_OK(hipGraphInstantiate(&g_graph, graph, NULL, NULL, 0));
    measure(do_accumulate, &dev[0], &host[0]);
    measure(do_copy, &dev[1], &host[1]);
    measure(do_rs_fused, &dev[2], &host[2]);
    measure(do_rs_steps, &dev[3], &host[3]);
    measure(do_rs_graph, &dev[4], &host[4]);
    measure(do_ag_fused, &dev[5], &host[5]);
    HIP_OK(hipGraphExecDestroy(g_graph));
    HIP_OK(hipGraphDestroy(graph));
    printf("%s{\"bytes\": %zu, \"accumulate_us\": %.2f, \"copy_us\": %.2f, \"ring_rs_p8_fused_us\": %.2f, "
           "\"ring_rs_p8_steps_us\": %.2f, \"ring_rs_p8_steps_graph_us\": %.2f, \"all_gather_p8_fused_us\": %.2f, "
           "\"host_us_accumulate\": %.2f, \"host_us_ring_rs_p8_fused\": %.2f, \"host_us_ring_rs_p8_steps\": %.2f, "
           "\"host_us_graph_launch\": %.2f}",
           bytes == 4096 ? "" : ", ", bytes, dev[0], dev[1], dev[2], dev[3], dev[4], dev[5], host[0], host[2], host[3],
           host[4]);
  }
  printf("]\n");
  return 0;
}
