/*
 * pccl_oracle.h -- plain-C restatement of PCCL's per-rank algorithms on host
 * buffers.  TEST INFRASTRUCTURE ONLY: linked by tests, by the smoke check and
 * by the CPU-baseline program, never by the product library.
 *
 * All ranks are simulated in one address space.  "in" is rank-major:
 * rank r's input starts at in + r * P * B elements; outputs likewise.
 * dtype: 0 = float32, 1 = bfloat16 bit patterns (uint16_t).
 */
#ifndef PCCL_ORACLE_H
#define PCCL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ORACLE_F32 = 0, ORACLE_BF16 = 1 };

/* a[i] += b[i] (pccl/src/common.cu:5-10). */
void oracle_vector_add_f32(float* a, const float* b, size_t n);
/* a[i] = bf16_rne(float(a[i]) + float(b[i])): torch.add on bfloat16. */
void oracle_vector_add_bf16(uint16_t* a, const uint16_t* b, size_t n);
void oracle_vector_add(void* a, const void* b, size_t n, int dtype);

uint16_t oracle_f32_to_bf16(float x);
float oracle_bf16_to_f32(uint16_t u);

/* pccl/src/reduce_scatter.cpp:101-155.  out: [P][B], in: [P][P*B]. */
int oracle_ring_reduce_scatter(void* out, const void* in, int P, size_t B, int dtype);
/* pccl/src/reduce_scatter.cpp:16-99.  P must be a power of two. */
int oracle_rh_reduce_scatter(void* out, const void* in, int P, size_t B, int dtype);
/* pccl/src/all_gather.cpp:15-69, bytes.  out: [P][P*blk], in: [P][blk]. */
int oracle_rd_all_gather(uint8_t* out, const uint8_t* in, int P, size_t blk);
/* Ring all_gather (schedule defined by this build), bytes. */
int oracle_ring_all_gather(uint8_t* out, const uint8_t* in, int P, size_t blk);

#ifdef __cplusplus
}
#endif
#endif
