/*
 * pccl_oracle.c -- plain-C CPU restatement of the reference's algorithms.
 * TEST INFRASTRUCTURE ONLY (see pccl_oracle.h).  Build without -ffast-math:
 * every add must stay one IEEE-754 RNE operation in the written order.
 *
 * Each collective simulates P ranks.  A rank has private work memory exactly
 * like the reference (d_buf / d_tmp, buf / recv_buf); one MPI_Sendrecv step is
 * "every rank copies its send region into the receiver's receive buffer, then
 * every rank reduces", which is what P simultaneous blocking Sendrecvs do.
 */
#include "pccl_oracle.h"

#include <stdlib.h>
#include <string.h>

float oracle_bf16_to_f32(uint16_t u) {
  uint32_t w = (uint32_t)u << 16;
  float f;
  memcpy(&f, &w, 4);
  return f;
}

uint16_t oracle_f32_to_bf16(float x) {
  uint32_t w;
  memcpy(&w, &x, 4);
  if ((w & 0x7fffffffu) > 0x7f800000u) return 0x7fc0; /* NaN -> canonical quiet NaN */
  w += 0x7fffu + ((w >> 16) & 1u);                     /* round to nearest, ties to even */
  return (uint16_t)(w >> 16);
}

/* pccl/src/common.cu:5-10: a[idx] += b[idx]. */
void oracle_vector_add_f32(float* a, const float* b, size_t n) {
  for (size_t i = 0; i < n; ++i) a[i] = a[i] + b[i];
}

/* torch.add on bfloat16 operands: widen, add in fp32, round once to bf16. */
void oracle_vector_add_bf16(uint16_t* a, const uint16_t* b, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float s = oracle_bf16_to_f32(a[i]) + oracle_bf16_to_f32(b[i]);
    a[i] = oracle_f32_to_bf16(s);
  }
}

void oracle_vector_add(void* a, const void* b, size_t n, int dtype) {
  if (dtype == ORACLE_F32) oracle_vector_add_f32((float*)a, (const float*)b, n);
  else oracle_vector_add_bf16((uint16_t*)a, (const uint16_t*)b, n);
}

static size_t esize(int dtype) { return dtype == ORACLE_F32 ? 4 : 2; }

/* pccl/src/reduce_scatter.cpp:101-155 */
int oracle_ring_reduce_scatter(void* out, const void* in, int P, size_t B, int dtype) {
  if (P < 1 || (dtype != ORACLE_F32 && dtype != ORACLE_BF16)) return -1;
  const size_t s = esize(dtype);
  const size_t total = (size_t)P * B;
  char* d_buf = (char*)malloc((size_t)P * total * s + 1);   /* per rank: total elems */
  char* d_tmp = (char*)malloc((size_t)P * B * s + 1);       /* per rank: one block   */
  if (!d_buf || !d_tmp) { free(d_buf); free(d_tmp); return -2; }
  memcpy(d_buf, in, (size_t)P * total * s);                  /* :119-123 */
  for (int step = 0; step < P - 1; ++step) {
    for (int rank = 0; rank < P; ++rank) {                   /* the sends of :140-142 */
      int send_idx = ((rank - step - 1) % P + P) % P;
      int dest = (rank + 1) % P;
      memcpy(d_tmp + (size_t)dest * B * s,
             d_buf + ((size_t)rank * total + (size_t)send_idx * B) * s, B * s);
    }
    for (int rank = 0; rank < P; ++rank) {                   /* :145 */
      int recv_idx = ((rank - step - 2) % P + P) % P;
      oracle_vector_add(d_buf + ((size_t)rank * total + (size_t)recv_idx * B) * s,
                        d_tmp + (size_t)rank * B * s, B, dtype);
    }
  }
  for (int rank = 0; rank < P; ++rank)                       /* :148-152 */
    memcpy((char*)out + (size_t)rank * B * s,
           d_buf + ((size_t)rank * total + (size_t)rank * B) * s, B * s);
  free(d_buf);
  free(d_tmp);
  return 0;
}

/* pccl/src/reduce_scatter.cpp:16-99 */
int oracle_rh_reduce_scatter(void* out, const void* in, int P, size_t B, int dtype) {
  if (P < 1 || (P & (P - 1)) || (dtype != ORACLE_F32 && dtype != ORACLE_BF16)) return -1;
  const size_t s = esize(dtype);
  const size_t total = (size_t)P * B;
  char* buf = (char*)malloc((size_t)P * total * s + 1);
  char* recv_buf = (char*)malloc((size_t)P * total * s + 1);
  size_t* curr = (size_t*)calloc((size_t)P, sizeof(size_t)); /* curr_ptr - buf, in elements */
  if (!buf || !recv_buf || !curr) { free(buf); free(recv_buf); free(curr); return -2; }
  memcpy(buf, in, (size_t)P * total * s);                    /* :32-36 */
  int rounds = 0;
  while ((1 << rounds) < P) ++rounds;                        /* :42 */
  int current_blocks = P;
  for (int r = 0; r < rounds; ++r) {
    int group_size = P / (1 << r);
    int half = current_blocks / 2;
    size_t count = (size_t)half * B;
    for (int rank = 0; rank < P; ++rank) {                   /* sends */
      int lower = (rank % group_size) < (group_size / 2);
      int partner = lower ? (rank + half) % P : (rank - half + P) % P;
      size_t send_off = lower ? curr[rank] + count : curr[rank];
      memcpy(recv_buf + (size_t)partner * total * s,
             buf + ((size_t)rank * total + send_off) * s, count * s);
    }
    for (int rank = 0; rank < P; ++rank) {                   /* :71 / :84-86 */
      int lower = (rank % group_size) < (group_size / 2);
      if (!lower) curr[rank] += count;
      oracle_vector_add(buf + ((size_t)rank * total + curr[rank]) * s,
                        recv_buf + (size_t)rank * total * s, count, dtype);
    }
    current_blocks = half;
  }
  for (int rank = 0; rank < P; ++rank)                       /* :92-96 */
    memcpy((char*)out + (size_t)rank * B * s,
           buf + ((size_t)rank * total + curr[rank]) * s, B * s);
  free(buf);
  free(recv_buf);
  free(curr);
  return 0;
}

/* pccl/src/all_gather.cpp:15-69 */
int oracle_rd_all_gather(uint8_t* out, const uint8_t* in, int P, size_t blk) {
  if (P < 1 || (P & (P - 1))) return -1;
  const size_t total = (size_t)P * blk;
  uint8_t* stage = (uint8_t*)malloc((size_t)P * total + 1); /* messages in flight */
  if (!stage) return -2;
  for (int rank = 0; rank < P; ++rank)                       /* :31-35 */
    memcpy(out + (size_t)rank * total + (size_t)rank * blk, in + (size_t)rank * blk, blk);
  for (int seg = 1; seg < P; seg *= 2) {
    size_t count = (size_t)seg * blk;
    for (int rank = 0; rank < P; ++rank) {                   /* sends of :61-63 */
      int partner = rank ^ seg;
      int group_start = (rank / (2 * seg)) * (2 * seg);
      size_t send_off = (rank < partner) ? (size_t)group_start * blk
                                         : (size_t)(group_start + seg) * blk;
      memcpy(stage + (size_t)partner * total, out + (size_t)rank * total + send_off, count);
    }
    for (int rank = 0; rank < P; ++rank) {                   /* receives */
      int partner = rank ^ seg;
      int group_start = (rank / (2 * seg)) * (2 * seg);
      size_t recv_off = (rank < partner) ? (size_t)(group_start + seg) * blk
                                         : (size_t)group_start * blk;
      memcpy(out + (size_t)rank * total + recv_off, stage + (size_t)rank * total, count);
    }
  }
  free(stage);
  return 0;
}

int oracle_ring_all_gather(uint8_t* out, const uint8_t* in, int P, size_t blk) {
  if (P < 1) return -1;
  const size_t total = (size_t)P * blk;
  uint8_t* stage = (uint8_t*)malloc((size_t)P * blk + 1);
  if (!stage) return -2;
  for (int rank = 0; rank < P; ++rank)
    memcpy(out + (size_t)rank * total + (size_t)rank * blk, in + (size_t)rank * blk, blk);
  for (int step = 0; step < P - 1; ++step) {
    for (int rank = 0; rank < P; ++rank) {
      int j = ((rank - step) % P + P) % P;
      int dest = (rank + 1) % P;
      memcpy(stage + (size_t)dest * blk, out + (size_t)rank * total + (size_t)j * blk, blk);
    }
    for (int rank = 0; rank < P; ++rank) {
      int j = ((rank - step - 1) % P + P) % P;
      memcpy(out + (size_t)rank * total + (size_t)j * blk, stage + (size_t)rank * blk, blk);
    }
  }
  free(stage);
  return 0;
}
