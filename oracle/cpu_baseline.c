/*
 * cpu_baseline.c -- the reference's ring / recursive-halving reduce_scatter run
 * as real processes on host cores, one process per rank.  TEST INFRASTRUCTURE
 * and CPU BASELINE ONLY: timed next to the GPU kernels, never shipped.
 *
 * Each rank executes the per-rank algorithm of pccl/src/reduce_scatter.cpp
 * (:101-155 ring, :16-99 recursive halving) on host buffers: copy the input to
 * the work buffer, then per step exchange one region with a neighbour
 * (MPI_Sendrecv) and add it with the scalar loop of pccl/src/common.cu:5-10.
 *
 * With -DUSE_MPI, "--alg mpi_block" times the vendor collective instead:
 * MPI_Reduce_scatter_block on float, what the reference reaches with
 * `--library mpi --pccl-disable-cpp-backend` (pccl/reduce_scatter.py:197).  Its
 * summation order belongs to the MPI library, so it is timed, not compared.
 *
 * Two transports, chosen at compile time:
 *   -DUSE_MPI : MPI_Sendrecv between MPI ranks (mpiexec -np P ...), the
 *               transport the reference uses;
 *   default   : fork() + an anonymous shared mapping + process-shared barriers,
 *               the same schedule where no MPI launcher is available
 *               (--ranks P selects the number of processes).
 *
 * Input of rank r, element i (seed s): u = splitmix64(s, r, i) >> 40 (24 bits),
 * x = (float)u / 2^23 - 1 in [-1, 1), times --scale; for bf16 then rounded RNE.
 * tests/ reproduce this generator in numpy to check the outputs bit for bit.
 *
 * Prints one JSON line on rank 0.  Timing follows
 * benchmark_raw_collectives/utils.py:16-33: warm-up calls, then the mean of the
 * timed calls; the slowest rank counts.
 */
#define _GNU_SOURCE
#include <errno.h>
#include <fcntl.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/wait.h>
#include <time.h>
#include <unistd.h>

#include "pccl_oracle.h"

#ifdef USE_MPI
#include <mpi.h>
#endif

typedef struct {
  int rank, size;
#ifndef USE_MPI
  char* mailbox;            /* [size][mail_bytes] shared */
  size_t mail_bytes;
  pthread_barrier_t* bar;   /* process-shared */
  double* times;            /* [size] shared */
#endif
} comm_t;

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static void comm_barrier(comm_t* c) {
#ifdef USE_MPI
  (void)c;
  MPI_Barrier(MPI_COMM_WORLD);
#else
  pthread_barrier_wait(c->bar);
#endif
}

/* Send `bytes` from sendp to `dest` and receive `bytes` from `src` into recvp. */
static void comm_sendrecv(comm_t* c, const void* sendp, int dest, void* recvp, int src,
                          size_t bytes, int tag) {
#ifdef USE_MPI
  (void)c;
  /* messages above INT_MAX bytes are split */
  size_t off = 0;
  while (off < bytes) {
    size_t chunk = bytes - off;
    if (chunk > (1u << 30)) chunk = 1u << 30;
    MPI_Sendrecv((const char*)sendp + off, (int)chunk, MPI_BYTE, dest, tag,
                 (char*)recvp + off, (int)chunk, MPI_BYTE, src, tag,
                 MPI_COMM_WORLD, MPI_STATUS_IGNORE);
    off += chunk;
  }
#else
  (void)src; (void)tag;
  memcpy(c->mailbox + (size_t)dest * c->mail_bytes, sendp, bytes);
  pthread_barrier_wait(c->bar);                     /* all messages delivered */
  memcpy(recvp, c->mailbox + (size_t)c->rank * c->mail_bytes, bytes);
  pthread_barrier_wait(c->bar);                     /* mailboxes free again   */
#endif
}

static double comm_max(comm_t* c, double v) {
#ifdef USE_MPI
  (void)c;
  double m;
  MPI_Allreduce(&v, &m, 1, MPI_DOUBLE, MPI_MAX, MPI_COMM_WORLD);
  return m;
#else
  c->times[c->rank] = v;
  pthread_barrier_wait(c->bar);
  double m = 0;
  for (int i = 0; i < c->size; ++i) if (c->times[i] > m) m = c->times[i];
  pthread_barrier_wait(c->bar);
  return m;
#endif
}

static uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

static void fill_input(void* buf, size_t n, int dtype, uint64_t seed, int rank, float scale) {
  uint64_t base = splitmix64(seed * 0x100000001B3ull + (uint64_t)rank);
  for (size_t i = 0; i < n; ++i) {
    uint32_t u = (uint32_t)(splitmix64(base + i) >> 40);
    float x = ((float)u / 8388608.0f - 1.0f) * scale;
    if (dtype == ORACLE_F32) ((float*)buf)[i] = x;
    else ((uint16_t*)buf)[i] = oracle_f32_to_bf16(x);
  }
}

/* pccl/src/reduce_scatter.cpp:101-155 on host buffers. */
static void ring_rs(comm_t* c, void* out, const void* in, size_t B, int dtype,
                    char* d_buf, char* d_tmp) {
  const int rank = c->rank, size = c->size;
  const size_t s = dtype == ORACLE_F32 ? 4 : 2;
  memcpy(d_buf, in, (size_t)size * B * s);
  for (int step = 0; step < size - 1; ++step) {
    int send_idx = ((rank - step - 1) % size + size) % size;
    int recv_idx = ((rank - step - 2) % size + size) % size;
    int dest = (rank + 1) % size;
    int source = (rank - 1 + size) % size;
    comm_sendrecv(c, d_buf + (size_t)send_idx * B * s, dest, d_tmp, source, B * s, 0);
    oracle_vector_add(d_buf + (size_t)recv_idx * B * s, d_tmp, B, dtype);
  }
  memcpy(out, d_buf + (size_t)rank * B * s, B * s);
}

/* pccl/src/reduce_scatter.cpp:16-99 on host buffers. */
static void rh_rs(comm_t* c, void* out, const void* in, size_t B, int dtype,
                  char* buf, char* recv_buf) {
  const int rank = c->rank, size = c->size;
  const size_t s = dtype == ORACLE_F32 ? 4 : 2;
  memcpy(buf, in, (size_t)size * B * s);
  int rounds = 0;
  while ((1 << rounds) < size) ++rounds;
  int current_blocks = size;
  char* curr = buf;
  for (int r = 0; r < rounds; ++r) {
    int group_size = size / (1 << r);
    int half = current_blocks / 2;
    size_t count = (size_t)half * B;
    if ((rank % group_size) < (group_size / 2)) {
      int partner = (rank + half) % size;
      comm_sendrecv(c, curr + count * s, partner, recv_buf, partner, count * s, r);
      oracle_vector_add(curr, recv_buf, count, dtype);
    } else {
      int partner = (rank - half + size) % size;
      comm_sendrecv(c, curr, partner, recv_buf, partner, count * s, r);
      curr += count * s;
      oracle_vector_add(curr, recv_buf, count, dtype);
    }
    current_blocks = half;
  }
  memcpy(out, curr, B * s);
}

typedef struct {
  const char* alg;
  int dtype;
  size_t B;
  int warmup, iters;
  uint64_t seed;
  float scale;
  const char* dump;
} opts_t;

static int run_rank(comm_t* c, const opts_t* o) {
  const size_t s = o->dtype == ORACLE_F32 ? 4 : 2;
  const size_t total = (size_t)c->size * o->B;
  void* in = malloc(total * s + 64);
  void* out = malloc(o->B * s + 64);
  char* w1 = (char*)malloc(total * s + 64);
  char* w2 = (char*)malloc(total * s + 64);
  if (!in || !out || !w1 || !w2) { fprintf(stderr, "rank %d: out of memory\n", c->rank); return 2; }
  fill_input(in, total, o->dtype, o->seed, c->rank, o->scale);
  double t0 = now_s();
  const int ring = strcmp(o->alg, "ring") == 0;
  const int vendor = strcmp(o->alg, "mpi_block") == 0;
  for (int i = 0; i < o->warmup + o->iters; ++i) {
    if (i == o->warmup) { comm_barrier(c); t0 = now_s(); }
#ifdef USE_MPI
    if (vendor) { MPI_Reduce_scatter_block(in, out, (int)o->B, MPI_FLOAT, MPI_SUM, MPI_COMM_WORLD); continue; }
#endif
    if (ring) ring_rs(c, out, in, o->B, o->dtype, w1, w2); else rh_rs(c, out, in, o->B, o->dtype, w1, w2);
  }
  (void)vendor;
  double dt = now_s() - t0;
  double worst = comm_max(c, dt);
  if (o->dump) {
    int fd = open(o->dump, O_WRONLY | O_CREAT, 0644);
    if (fd < 0 || pwrite(fd, out, o->B * s, (off_t)((size_t)c->rank * o->B * s)) != (ssize_t)(o->B * s)) {
      fprintf(stderr, "rank %d: cannot write %s: %s\n", c->rank, o->dump, strerror(errno));
      return 3;
    }
    close(fd);
  }
  if (c->rank == 0) {
    double ms = o->iters ? 1e3 * worst / o->iters : 0.0;
    /* algorithmic bytes of the whole job: every rank adds (P-1) regions of B
     * elements, 2 reads + 1 write each */
    double bytes = 3.0 * (double)(c->size - 1) * (double)o->B * (double)s * (double)c->size;
    printf("{\"transport\": \"%s\", \"algorithm\": \"%s\", \"ranks\": %d, \"dtype\": \"%s\", "
           "\"block_elems\": %zu, \"warmup\": %d, \"iters\": %d, \"ms_per_call\": %.6f, "
           "\"algorithmic_bytes\": %.0f, \"GBps\": %.6f}\n",
#ifdef USE_MPI
           "mpi",
#else
           "fork+shm",
#endif
           o->alg, c->size, o->dtype == ORACLE_F32 ? "f32" : "bf16", o->B, o->warmup, o->iters,
           ms, bytes, ms > 0 ? bytes / (ms * 1e-3) / 1e9 : 0.0);
    fflush(stdout);
  }
  free(in); free(out); free(w1); free(w2);
  return 0;
}

int main(int argc, char** argv) {
  opts_t o = {"ring", ORACLE_F32, 1 << 20, 1, 3, 1234, 1.0f, NULL};
  int ranks = 4;
  for (int i = 1; i < argc; ++i) {
    const char* a = argv[i];
    const char* v = (i + 1 < argc) ? argv[i + 1] : "";
    if (!strcmp(a, "--alg")) { o.alg = v; ++i; }
    else if (!strcmp(a, "--dtype")) { o.dtype = strcmp(v, "bf16") ? ORACLE_F32 : ORACLE_BF16; ++i; }
    else if (!strcmp(a, "--block")) { o.B = (size_t)strtoull(v, NULL, 10); ++i; }
    else if (!strcmp(a, "--ranks")) { ranks = atoi(v); ++i; }
    else if (!strcmp(a, "--warmup")) { o.warmup = atoi(v); ++i; }
    else if (!strcmp(a, "--iters")) { o.iters = atoi(v); ++i; }
    else if (!strcmp(a, "--seed")) { o.seed = strtoull(v, NULL, 10); ++i; }
    else if (!strcmp(a, "--scale")) { o.scale = strtof(v, NULL); ++i; }
    else if (!strcmp(a, "--dump")) { o.dump = v; ++i; }
    else { fprintf(stderr, "unknown argument %s\n", a); return 64; }
  }
  if (strcmp(o.alg, "ring") && strcmp(o.alg, "recursive") && strcmp(o.alg, "mpi_block")) {
    fprintf(stderr, "--alg must be ring, recursive or mpi_block\n");
    return 64;
  }
#ifndef USE_MPI
  if (!strcmp(o.alg, "mpi_block")) { fprintf(stderr, "--alg mpi_block needs the MPI build\n"); return 64; }
#endif
  if (!strcmp(o.alg, "mpi_block") && o.dtype != ORACLE_F32) {
    fprintf(stderr, "--alg mpi_block is float only (MPI has no bfloat16)\n");
    return 64;
  }
#ifdef USE_MPI
  (void)ranks;
  MPI_Init(&argc, &argv);
  comm_t c;
  MPI_Comm_rank(MPI_COMM_WORLD, &c.rank);
  MPI_Comm_size(MPI_COMM_WORLD, &c.size);
  if (strcmp(o.alg, "recursive") == 0 && (c.size & (c.size - 1))) {
    if (c.rank == 0) fprintf(stderr, "recursive halving needs a power-of-two number of ranks\n");
    MPI_Finalize();
    return 64;
  }
  int rc = run_rank(&c, &o);
  MPI_Finalize();
  return rc;
#else
  if (ranks < 1 || ranks > 256) { fprintf(stderr, "--ranks out of range\n"); return 64; }
  if (strcmp(o.alg, "recursive") == 0 && (ranks & (ranks - 1))) {
    fprintf(stderr, "recursive halving needs a power-of-two number of ranks\n");
    return 64;
  }
  const size_t s = o.dtype == ORACLE_F32 ? 4 : 2;
  /* ring sends one block per step, halving at most half the buffer */
  size_t mail = (strcmp(o.alg, "ring") == 0 ? o.B : (size_t)ranks * o.B / 2 + 1) * s;
  mail = (mail + 4095) & ~(size_t)4095;
  size_t ctl = 4096 + sizeof(double) * (size_t)ranks;
  ctl = (ctl + 4095) & ~(size_t)4095;
  char* shm = (char*)mmap(NULL, ctl + mail * (size_t)ranks, PROT_READ | PROT_WRITE,
                          MAP_SHARED | MAP_ANONYMOUS, -1, 0);
  if (shm == MAP_FAILED) { perror("mmap"); return 2; }
  pthread_barrier_t* bar = (pthread_barrier_t*)shm;
  pthread_barrierattr_t at;
  pthread_barrierattr_init(&at);
  pthread_barrierattr_setpshared(&at, PTHREAD_PROCESS_SHARED);
  pthread_barrier_init(bar, &at, (unsigned)ranks);
  if (o.dump) { int fd = open(o.dump, O_WRONLY | O_CREAT | O_TRUNC, 0644); if (fd >= 0) close(fd); }
  pid_t* pids = (pid_t*)calloc((size_t)ranks, sizeof(pid_t));
  for (int r = 0; r < ranks; ++r) {
    pid_t p = fork();
    if (p < 0) { perror("fork"); return 2; }
    if (p == 0) {
      comm_t c;
      c.rank = r; c.size = ranks;
      c.mailbox = shm + ctl; c.mail_bytes = mail; c.bar = bar;
      c.times = (double*)(shm + 4096);
      _exit(run_rank(&c, &o));
    }
    pids[r] = p;
  }
  int rc = 0;
  for (int r = 0; r < ranks; ++r) {
    int st = 0;
    waitpid(pids[r], &st, 0);
    if (!WIFEXITED(st) || WEXITSTATUS(st)) rc = 1;
  }
  free(pids);
  return rc;
#endif
}
