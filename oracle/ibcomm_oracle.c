/*
 * CPU oracle for the PFNProto allreduce hot path -- TEST INFRASTRUCTURE ONLY.
 * See ibcomm_oracle.h for what this is, who may call it, and how each function
 * is pinned.  Citations are paths relative to the reference checkout.
 *
 * Structure: one pthread per emulated rank runs a restatement of the
 * reference's per-rank routine.  "Device" operations of the GPU schedules are
 * executed synchronously on host memory (a stream is always idle when
 * queried), the InfiniBand queue pairs are replaced by an in-memory FIFO
 * channel per ordered pair of ranks with the semantics the schedules rely on:
 * the k-th send A->B is delivered into the k-th buffer B posted for A, posts
 * never block, polls report each completion once.
 */
#define _GNU_SOURCE
#include "ibcomm_oracle.h"

#include <limits.h>
#include <pthread.h>
#include <sched.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ------------------------------------------------------------------------ */
/* util.h                                                                   */
/* ------------------------------------------------------------------------ */

size_t orc_dtype_size(int dtype) {
  switch (dtype) {
    case ORC_F32: case ORC_I32: return 4;
    case ORC_F64: case ORC_I64: return 8;
    default: return 0;
  }
}

/* util.h:151-154 */
int64_t orc_ceil_div(int64_t v1, int64_t v2) {
  return (v1 % v2) ? v1 / v2 + 1 : v1 / v2;
}

/* util.h:156-175: exponent p with 2^p == n, and 0 for anything that is not a
 * power of two -- which makes n == 1 indistinguishable from "not a power". */
int orc_get_exp_of_two(int n) {
  int p = 0;
  while (n != 0) {
    if (n % 2 == 1) return (n == 1) ? p : 0;
    p++;
    n >>= 1;
  }
  return 0;
}

/* ------------------------------------------------------------------------ */
/* partitioning: ibverbs_communicator.cpp:618-707                            */
/* ------------------------------------------------------------------------ */

int orc_read_chunk_size(const char* env, int* out_bytes) {
  if (env == NULL) { *out_bytes = -1; return ORC_OK; }
  int v = atoi(env);                       /* :623 */
  if (v <= 0) return ORC_INVALID_ARGUMENT; /* :625-628 */
  *out_bytes = v;
  return ORC_OK;
}

int orc_split_buffer(size_t len_elements, size_t sizeof_element, int world_size,
                     const char* env_chunksize, size_t* starts, size_t* ends,
                     int cap, int* n_ranges) {
  long chunks;
  size_t elements_per_chunk;
  *n_ranges = 0;

  if (len_elements < (size_t)world_size) return ORC_NOT_SUPPORTED; /* :642-648 */

  int env_bytes;
  int rc = orc_read_chunk_size(env_chunksize, &env_bytes);         /* :650 */
  if (rc != ORC_OK) return rc;

  if (env_bytes != -1) {
    if ((size_t)env_bytes % sizeof_element != 0) return ORC_INVALID_ARGUMENT; /* :653-657 */
    elements_per_chunk = (size_t)env_bytes / sizeof_element;                 /* :659 */
    chunks = (long)orc_ceil_div((int64_t)len_elements, (int64_t)elements_per_chunk);
    if (chunks < 2L * world_size) return ORC_INVALID_ARGUMENT;               /* :662-668 */
  } else {
    chunks = 4L * world_size;                                                /* :670 */
    elements_per_chunk = (size_t)orc_ceil_div((int64_t)len_elements, chunks);
  }

  /* :675-680.  The reference keeps start/end in `int`; every configuration it
   * is exercised with stays below INT_MAX, where size_t gives the same
   * ranges.  Empty trailing ranges are dropped. */
  int n = 0;
  for (long i = 0; i < chunks; i++) {
    size_t s = elements_per_chunk * (size_t)i;
    size_t e = elements_per_chunk * (size_t)(i + 1);
    if (e > len_elements) e = len_elements;
    if (s < e) {
      if (n < cap) { starts[n] = s; ends[n] = e; }
      n++;
    }
  }
  *n_ranges = n;
  return (n <= cap) ? ORC_OK : ORC_INTERNAL;
}

void orc_rank_to_chunk(int n_ranges, int world_size, int* first_chunk,
                       int* n_chunks) {
  int per = n_ranges / world_size;  /* :688 */
  int rem = n_ranges % world_size;  /* :689 */
  int id = 0;
  for (int i = 0; i < world_size; i++) {
    first_chunk[i] = id;
    n_chunks[i] = per + (i < rem ? 1 : 0); /* :693-701 */
    id += n_chunks[i];
  }
}

/* ------------------------------------------------------------------------ */
/* the reduction loop: allreduce_cpu_impl.h:16-21                            */
/* ------------------------------------------------------------------------ */

static void reduce_f32(float* result, const float* value, size_t n) {
  for (size_t i = 0; i < n; i++) result[i] += value[i];
}
static void reduce_f64(double* result, const double* value, size_t n) {
  for (size_t i = 0; i < n; i++) result[i] += value[i];
}
/* integer += wraps in the reference's generated code; spell it unsigned so
 * that it is defined behaviour here. */
static void reduce_u32(uint32_t* result, const uint32_t* value, size_t n) {
  for (size_t i = 0; i < n; i++) result[i] += value[i];
}
static void reduce_u64(uint64_t* result, const uint64_t* value, size_t n) {
  for (size_t i = 0; i < n; i++) result[i] += value[i];
}

void orc_reduce_inplace(int dtype, void* result, const void* value, size_t n) {
  switch (dtype) {
    case ORC_F32: reduce_f32((float*)result, (const float*)value, n); break;
    case ORC_I32: reduce_u32((uint32_t*)result, (const uint32_t*)value, n); break;
    case ORC_F64: reduce_f64((double*)result, (const double*)value, n); break;
    case ORC_I64: reduce_u64((uint64_t*)result, (const uint64_t*)value, n); break;
    default: break;
  }
}

/* ------------------------------------------------------------------------ */
/* small FIFO containers                                                    */
/* ------------------------------------------------------------------------ */

typedef struct { int range_id, depth, pair_rank, reduce, last; } chunk_t; /* allreduce_cuda_impl.h:303-324 */

#define DEFINE_QUEUE(NAME, T)                                              \
  typedef struct { T* v; long head, tail, cap; } NAME;                     \
  __attribute__((unused)) static void NAME##_push(NAME* q, T x) {                                  \
    if (q->tail == q->cap) {                                               \
      long live = q->tail - q->head;                                       \
      if (q->head > 0 && live <= q->cap / 2) {                             \
        memmove(q->v, q->v + q->head, (size_t)live * sizeof(T));           \
      } else {                                                             \
        long ncap = q->cap ? q->cap * 2 : 16;                              \
        T* nv = (T*)malloc((size_t)ncap * sizeof(T));                      \
        if (live) memcpy(nv, q->v + q->head, (size_t)live * sizeof(T));    \
        free(q->v);                                                        \
        q->v = nv;                                                         \
        q->cap = ncap;                                                     \
      }                                                                    \
      q->head = 0;                                                         \
      q->tail = live;                                                      \
    }                                                                      \
    q->v[q->tail++] = x;                                                   \
  }                                                                        \
  __attribute__((unused)) static int NAME##_empty(const NAME* q) { return q->head == q->tail; }    \
  __attribute__((unused)) static long NAME##_size(const NAME* q) { return q->tail - q->head; }     \
  __attribute__((unused)) static T NAME##_front(const NAME* q) { return q->v[q->head]; }           \
  __attribute__((unused)) static T NAME##_pop(NAME* q) { return q->v[q->head++]; }                 \
  __attribute__((unused)) static void NAME##_free(NAME* q) { free(q->v); q->v = NULL; q->head = q->tail = q->cap = 0; }

typedef struct { const char* ptr; size_t bytes; size_t log_off; } post_t;
typedef char* slot_t;

DEFINE_QUEUE(iq, int)
DEFINE_QUEUE(cq, chunk_t)
DEFINE_QUEUE(pq, post_t)
DEFINE_QUEUE(sq, slot_t)

/* ------------------------------------------------------------------------ */
/* loopback "network"                                                       */
/* ------------------------------------------------------------------------ */

typedef struct {
  pthread_mutex_t mu;
  pq sends, recvs;         /* posted, not yet matched */
  long send_done;          /* completions the sender has not polled yet */
  long recv_done;          /* completions the receiver has not polled yet */
  size_t* log_off;
  size_t* log_n;
  long log_count, log_cap;
} channel_t;

typedef struct {
  int n;
  int dtype;
  size_t esize;
  channel_t* ch;           /* n*n, [src*n + dst] */
  volatile int abort_flag; /* set on watchdog expiry or internal error */
  double deadline;         /* CLOCK_MONOTONIC seconds */
  long messages;
} world_t;

static double now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static int world_dead(world_t* w) {
  if (w->abort_flag) return 1;
  if (now_s() > w->deadline) { w->abort_flag = 1; return 1; }
  return 0;
}

static void channel_match(world_t* w, channel_t* c) {
  while (!pq_empty(&c->sends) && !pq_empty(&c->recvs)) {
    post_t s = pq_pop(&c->sends);
    post_t r = pq_pop(&c->recvs);
    if (s.bytes != r.bytes) { w->abort_flag = 1; return; }
    memcpy((char*)r.ptr, s.ptr, s.bytes);
    if (c->log_count == c->log_cap) {
      c->log_cap = c->log_cap ? c->log_cap * 2 : 64;
      c->log_off = (size_t*)realloc(c->log_off, (size_t)c->log_cap * sizeof(size_t));
      c->log_n = (size_t*)realloc(c->log_n, (size_t)c->log_cap * sizeof(size_t));
    }
    c->log_off[c->log_count] = s.log_off;
    c->log_n[c->log_count] = s.bytes / w->esize;
    c->log_count++;
    c->send_done++;
    c->recv_done++;
    __sync_fetch_and_add(&w->messages, 1);
  }
}

/* SendRegistered(dest, buf, mr, len, false): ibverbs_communicator.cpp:386-414 */
static void net_send(world_t* w, int me, int dest, const void* buf, size_t bytes, size_t log_off) {
  channel_t* c = &w->ch[me * w->n + dest];
  post_t p = {(const char*)buf, bytes, log_off};
  pthread_mutex_lock(&c->mu);
  pq_push(&c->sends, p);
  channel_match(w, c);
  pthread_mutex_unlock(&c->mu);
}

/* RecvRegistered(src, buf, mr, len, false): ibverbs_communicator.cpp:501-527 */
static void net_recv(world_t* w, int me, int src, void* buf, size_t bytes) {
  channel_t* c = &w->ch[src * w->n + me];
  post_t p = {(const char*)buf, bytes, 0};
  pthread_mutex_lock(&c->mu);
  pq_push(&c->recvs, p);
  channel_match(w, c);
  pthread_mutex_unlock(&c->mu);
}

/* SendPoll: ibverbs_communicator.cpp:416-461 */
static int net_send_poll(world_t* w, int me, int dest) {
  channel_t* c = &w->ch[me * w->n + dest];
  int ok = 0;
  pthread_mutex_lock(&c->mu);
  if (c->send_done > 0) { c->send_done--; ok = 1; }
  pthread_mutex_unlock(&c->mu);
  return ok;
}

/* RecvPoll: ibverbs_communicator.cpp:529-572 */
static int net_recv_poll(world_t* w, int me, int src) {
  channel_t* c = &w->ch[src * w->n + me];
  int ok = 0;
  pthread_mutex_lock(&c->mu);
  if (c->recv_done > 0) { c->recv_done--; ok = 1; }
  pthread_mutex_unlock(&c->mu);
  return ok;
}

/* SendWait / RecvWait: ibverbs_communicator.cpp:463-473, 574-584.  Returns 0
 * when the watchdog fired instead. */
static int net_send_wait(world_t* w, int me, int dest) {
  while (!net_send_poll(w, me, dest)) { if (world_dead(w)) return 0; sched_yield(); }
  return 1;
}
static int net_recv_wait(world_t* w, int me, int src) {
  while (!net_recv_poll(w, me, src)) { if (world_dead(w)) return 0; sched_yield(); }
  return 1;
}

/* ------------------------------------------------------------------------ */
/* staging pool: memory_pool.h:191-273                                      */
/* ------------------------------------------------------------------------ */

typedef struct {
  size_t block_bytes, chunk_bytes;
  char** blocks;
  int n_blocks;
  sq vacant;               /* vacant_memories_, FIFO */
  int held, high_water;
  int failed;              /* chunk does not fit a block: reference pops an empty queue */
} pool_t;

static void pool_add_block(pool_t* p) {
  p->blocks = (char**)realloc(p->blocks, (size_t)(p->n_blocks + 1) * sizeof(char*));
  char* b = (char*)malloc(p->block_bytes);
  p->blocks[p->n_blocks++] = b;
  /* memory_pool.h:269-271: strict '<', so a block of exactly k chunks yields k-1 slots */
  for (size_t i = 0; (i + 1) * p->chunk_bytes < p->block_bytes; i++) sq_push(&p->vacant, b + i * p->chunk_bytes);
}

/* MemoryPool ctor pre-allocates one block (memory_pool.h:99); GetController
 * carves every existing block (:208-210). */
static void pool_init(pool_t* p, size_t block_bytes, size_t chunk_bytes) {
  memset(p, 0, sizeof(*p));
  p->block_bytes = block_bytes;
  p->chunk_bytes = chunk_bytes;
  pool_add_block(p);
}

/* MemoryController::getMemory, memory_pool.h:222-236 */
static char* pool_get(pool_t* p) {
  if (sq_empty(&p->vacant)) pool_add_block(p);
  if (sq_empty(&p->vacant)) { p->failed = 1; return NULL; }
  char* s = sq_pop(&p->vacant);
  p->held++;
  if (p->held > p->high_water) p->high_water = p->held;
  return s;
}

/* MemoryController::returnMemory, memory_pool.h:238-242 */
static void pool_put(pool_t* p, char* s) {
  sq_push(&p->vacant, s);
  p->held--;
}

static void pool_destroy(pool_t* p) {
  for (int i = 0; i < p->n_blocks; i++) free(p->blocks[i]);
  free(p->blocks);
  sq_free(&p->vacant);
}

/* ------------------------------------------------------------------------ */
/* per-rank state                                                           */
/* ------------------------------------------------------------------------ */

typedef struct {
  world_t* w;
  int rank;
  int algo;
  const char* sendbuf;
  char* recvbuf;
  size_t len;
  const char* env_chunk;
  size_t pool_block;
  int rc;
  int pool_high_water, pool_blocks, slots_leaked;
} rank_t;

typedef struct {
  int n_ranges;
  size_t* starts;
  size_t* ends;
  int* first;  /* rank -> first chunk id */
  int* count;  /* rank -> chunk count */
} part_t;

static int part_build(part_t* P, size_t len, size_t esize, int N, const char* env) {
  memset(P, 0, sizeof(*P));
  /* upper bound on the number of ranges: env chunk of one element -> len ranges; default -> 4N */
  int cap_try = 4 * N;
  int env_bytes;
  int rc = orc_read_chunk_size(env, &env_bytes);
  if (rc != ORC_OK) {
    /* SplitBuffer checks the length first (:642) and the variable second (:650) */
    if (len < (size_t)N) return ORC_NOT_SUPPORTED;
    return rc;
  }
  if (env_bytes != -1 && (size_t)env_bytes >= esize) {
    size_t epc = (size_t)env_bytes / esize;
    size_t c = (len + epc - 1) / epc;
    if (c > (size_t)INT_MAX / 2) return ORC_INTERNAL;
    if ((int)c > cap_try) cap_try = (int)c;
  }
  P->starts = (size_t*)malloc((size_t)cap_try * sizeof(size_t));
  P->ends = (size_t*)malloc((size_t)cap_try * sizeof(size_t));
  rc = orc_split_buffer(len, esize, N, env, P->starts, P->ends, cap_try, &P->n_ranges);
  if (rc != ORC_OK) return rc;
  P->first = (int*)malloc((size_t)N * sizeof(int));
  P->count = (int*)malloc((size_t)N * sizeof(int));
  orc_rank_to_chunk(P->n_ranges, N, P->first, P->count);
  return ORC_OK;
}

static void part_free(part_t* P) {
  free(P->starts); free(P->ends); free(P->first); free(P->count);
  memset(P, 0, sizeof(*P));
}

#define OFF(i)   (P.starts[(i)])
#define NEL(i)   (P.ends[(i)] - P.starts[(i)])
#define BOFF(i)  (OFF(i) * es)
#define BYTES(i) (NEL(i) * es)

/* ------------------------------------------------------------------------ */
/* AllreduceRing<T>, allreduce_cpu_impl.h:23-244                             */
/* Memory-region bookkeeping (mrs, send_mrs, recv_mrs) moves no data and is  */
/* left out; everything that orders sends, receives and reductions is kept.  */
/* ------------------------------------------------------------------------ */

static void ring_cpu(rank_t* R) {
  world_t* w = R->w;
  const int N = w->n, r = R->rank;
  const size_t es = w->esize;
  if (N == 1) { memcpy(R->recvbuf, R->sendbuf, es * R->len); return; }  /* :26-29 */

  part_t P;
  R->rc = part_build(&P, R->len, es, N, R->env_chunk);                 /* :31-32 */
  if (R->rc) { part_free(&P); return; }
  const int chunks = P.n_ranges;
  const int from = (r - 1 + N) % N, to = (r + 1) % N;                   /* :36-37 */

  iq reg_q = {0}, first_send_q = {0}, buffering = {0};
  for (int i = 0; i < N - 1; i++) {                                     /* :40-48 */
    int g = (r - i - 1 + N) % N;
    for (int c = P.first[g] + P.count[g] - 1; c >= P.first[g]; c--) iq_push(&reg_q, c);
  }
  for (int c = P.first[r] + P.count[r] - 1; c >= P.first[r]; c--) iq_push(&first_send_q, c); /* :66-69 */

  int send_q_elements = 0, recv_q_elements = 0;
  int cur = iq_front(&reg_q);                                           /* :71 */
  int reduce_scatter_done = 0;
  const int to_front = P.first[to], to_back = P.first[to] + P.count[to] - 1;

  while (!reduce_scatter_done) {                                        /* :75 */
    if (world_dead(w)) goto out;
    while ((iq_empty(&reg_q) || recv_q_elements > 0) && net_recv_poll(w, r, from)) { /* :76 */
      recv_q_elements--;
      orc_reduce_inplace(w->dtype, R->recvbuf + BOFF(cur), R->sendbuf + BOFF(cur), NEL(cur)); /* :84-85 */
      if (cur == to_front) reduce_scatter_done = 1;                     /* :87-89 */
      if (!(to_front <= cur && cur <= to_back)) {                       /* :91-100 */
        if (iq_empty(&first_send_q) && iq_empty(&buffering)) {
          net_send(w, r, to, R->recvbuf + BOFF(cur), BYTES(cur), OFF(cur));
          send_q_elements++;
        } else {
          iq_push(&buffering, cur);
        }
      }
      cur = (cur - 1 + chunks) % chunks;                                /* :102 */
    }
    if (!iq_empty(&reg_q)) {                                            /* :105-119 */
      int k = iq_pop(&reg_q);
      net_recv(w, r, from, R->recvbuf + BOFF(k), BYTES(k));
      recv_q_elements++;
    }
    if (!iq_empty(&first_send_q)) {                                     /* :121-135 */
      int i = iq_pop(&first_send_q);
      net_send(w, r, to, R->sendbuf + BOFF(i), BYTES(i), OFF(i));
      send_q_elements++;
    } else {
      while (!iq_empty(&buffering)) {                                   /* :137-149 */
        int i = iq_pop(&buffering);
        net_send(w, r, to, R->recvbuf + BOFF(i), BYTES(i), OFF(i));
        send_q_elements++;
      }
    }
    while (net_send_poll(w, r, to)) send_q_elements--;                  /* :152-157 */
    sched_yield();
  }

  while (send_q_elements != 0) {                                        /* :177-184 */
    if (!net_send_wait(w, r, to)) goto out;
    send_q_elements--;
  }

  for (int i = 0; i < N; i++) {                                         /* :187-225 */
    int g = (1 + r - i + N) % N;
    for (int c = P.first[g] + P.count[g] - 1; c >= P.first[g]; c--) {
      if (g != (r + 1) % N) {
        net_recv(w, r, from, R->recvbuf + BOFF(c), BYTES(c));
        while (!net_recv_poll(w, r, from)) {
          if (world_dead(w)) goto out;
          if (net_send_poll(w, r, to)) send_q_elements--;
          else sched_yield();
        }
      }
      if (g != (r + 2) % N) {
        net_send(w, r, to, R->recvbuf + BOFF(c), BYTES(c), OFF(c));
        send_q_elements++;
      }
    }
  }
  while (send_q_elements != 0) {                                        /* :227-234 */
    if (!net_send_wait(w, r, to)) goto out;
    send_q_elements--;
  }
out:
  iq_free(&reg_q); iq_free(&first_send_q); iq_free(&buffering);
  part_free(&P);
}

/* ------------------------------------------------------------------------ */
/* AllreduceRabenseifner<T>, allreduce_cpu_impl.h:246-372                    */
/* Un-chunked: N ranges of ceilDiv(len, N), one message per step.            */
/* ------------------------------------------------------------------------ */

static void raben_cpu(rank_t* R) {
  world_t* w = R->w;
  const int N = w->n, r = R->rank;
  const size_t es = w->esize;
  if (N == 1) { memcpy(R->recvbuf, R->sendbuf, es * R->len); return; }  /* :249-252 */
  const int exp = orc_get_exp_of_two(N);
  if (exp == 0) { R->rc = ORC_NOT_SUPPORTED; return; }                 /* :254-262 */

  /* :264-271.  When range_length * i exceeds len for some i the reference
   * builds an inverted range and its size_t arithmetic wraps; that input is
   * outside what the reference defines, so it is refused here. */
  const size_t rl = (size_t)orc_ceil_div((int64_t)R->len, N);
  if (rl * (size_t)(N - 1) > R->len) { R->rc = ORC_NOT_SUPPORTED; return; }
  size_t* first = (size_t*)malloc((size_t)N * sizeof(size_t));
  size_t* second = (size_t*)malloc((size_t)N * sizeof(size_t));
  for (int i = 0; i < N; i++) {
    first[i] = rl * (size_t)i;
    second[i] = rl * (size_t)(i + 1) < R->len ? rl * (size_t)(i + 1) : R->len;
  }
  char* tmp = (char*)malloc(es * R->len);                               /* :273 */
  memcpy(R->recvbuf, R->sendbuf, es * R->len);                          /* :279 */

  int start = 0, end = N;
  for (int step = 0; step < exp; step++) {                              /* :285-329 */
    int to = r ^ (1 << step);
    int ss, se, rs, re;
    if (r < to) { ss = start; se = end - (end - start) / 2; rs = se; re = end; }
    else        { rs = start; re = end - (end - start) / 2; ss = re; se = end; }
    size_t sn = second[(se - 1 + N) % N] - first[ss];
    size_t rn = second[(re - 1 + N) % N] - first[rs];
    net_send(w, r, to, R->recvbuf + first[ss] * es, sn * es, first[ss]);
    net_recv(w, r, to, tmp + first[rs] * es, rn * es);
    if (!net_recv_wait(w, r, to)) goto out;
    orc_reduce_inplace(w->dtype, R->recvbuf + first[rs] * es, tmp + first[rs] * es, rn); /* :319-323 */
    if (!net_send_wait(w, r, to)) goto out;
    start = rs; end = re;
  }
  for (int step = 0; step < exp; step++) {                              /* :332-369 */
    int to = r ^ (1 << (exp - step - 1));
    int ss = start, se = end, rs, re;
    if (r > to) { rs = se; re = rs + end - start; }
    else        { re = ss; rs = re - (end - start); }
    size_t sn = second[(se - 1 + N) % N] - first[ss];
    size_t rn = second[(re - 1 + N) % N] - first[rs];
    net_send(w, r, to, R->recvbuf + first[ss] * es, sn * es, first[ss]);
    net_recv(w, r, to, R->recvbuf + first[rs] * es, rn * es);
    if (!net_recv_wait(w, r, to)) goto out;
    if (!net_send_wait(w, r, to)) goto out;
    start = ss < rs ? ss : rs;
    end = se > re ? se : re;
  }
out:
  free(tmp); free(first); free(second);
}

/* ------------------------------------------------------------------------ */
/* AllreduceRingCuda<T>, allreduce_cuda_impl.h:35-301                        */
/* cudaMemcpyAsync / kernel launches run synchronously here, so every        */
/* cudaStreamQuery would answer "idle" and every cudaStreamSynchronize is a  */
/* no-op.                                                                    */
/* ------------------------------------------------------------------------ */

static void ring_gpu(rank_t* R) {
  world_t* w = R->w;
  const int N = w->n, r = R->rank;
  const size_t es = w->esize;
  if (N == 1) { memcpy(R->recvbuf, R->sendbuf, es * R->len); return; }  /* :40-46 */

  part_t P;
  R->rc = part_build(&P, R->len, es, N, R->env_chunk);                 /* :48-49 */
  if (R->rc) { part_free(&P); return; }
  const int chunks = P.n_ranges;
  const int from = (r - 1 + N) % N, to = (r + 1) % N;                   /* :53-54 */

  pool_t pool;
  pool_init(&pool, R->pool_block, BYTES(0));                            /* :56-57 */
  char** mem = (char**)calloc((size_t)chunks, sizeof(char*));           /* :59 */

  iq reg_q = {0}, first_send_q = {0}, buffering = {0};
  iq wait_send_q = {0}, wait_reduction_q = {0}, wait_send_completion_q = {0};
  for (int i = 0; i < N - 1; i++) {                                     /* :63-71 */
    int g = (r - i - 1 + N) % N;
    for (int c = P.first[g] + P.count[g] - 1; c >= P.first[g]; c--) iq_push(&reg_q, c);
  }
  for (int i = 0; i < N - 1; i++) {                                     /* :74-81 */
    int g = (r - i + N) % N;
    for (int c = P.first[g] + P.count[g] - 1; c >= P.first[g]; c--) iq_push(&reg_q, c);
  }
  for (int c = P.first[r] + P.count[r] - 1; c >= P.first[r]; c--) iq_push(&first_send_q, c); /* :86-89 */

  int cur = iq_front(&reg_q);                                           /* :91 */
  int remaining_recv_q_length = 0;
  int reduce_scatter_phase = 1;
  const int final_rank = (r + 2) % N;                                   /* :99 */
  const int fin_front = P.first[final_rank], fin_back = P.first[final_rank] + P.count[final_rank] - 1;

  for (;;) {                                                            /* :103 */
    if (world_dead(w) || pool.failed) break;
    while ((reduce_scatter_phase || iq_empty(&wait_reduction_q)) && net_recv_poll(w, r, from)) { /* :104-105 */
      remaining_recv_q_length--;
      char* m = mem[cur];
      memcpy(R->recvbuf + BOFF(cur), m, BYTES(cur));                    /* :129-130 */
      if (reduce_scatter_phase) {
        orc_reduce_inplace(w->dtype, R->recvbuf + BOFF(cur), R->sendbuf + BOFF(cur), NEL(cur)); /* :132-133 */
        memcpy(m, R->recvbuf + BOFF(cur), BYTES(cur));                  /* :134-135 */
        iq_push(&wait_reduction_q, cur);
        if (cur == P.first[to]) reduce_scatter_phase = 0;               /* :137-139 */
      } else {
        if (cur < fin_front || fin_back < cur) {                        /* :144-151 */
          net_send(w, r, to, m, BYTES(cur), OFF(cur));
          iq_push(&wait_send_completion_q, cur);
        } else {                                                        /* :152-157 */
          pool_put(&pool, m);
          mem[cur] = NULL;
        }
      }
      cur = (cur - 1 + chunks) % chunks;                                /* :159 */
    }

    if (!reduce_scatter_phase && iq_empty(&wait_reduction_q) &&
        cur == (fin_front - 1 + chunks) % chunks) break;                /* :164-167 */

    if (!iq_empty(&wait_reduction_q)) {                                 /* :169-196 */
      int i = iq_pop(&wait_reduction_q);
      if (iq_empty(&first_send_q) && iq_empty(&wait_send_q) && iq_empty(&buffering)) {
        net_send(w, r, to, mem[i], BYTES(i), OFF(i));
        iq_push(&wait_send_completion_q, i);
      } else {
        iq_push(&buffering, i);
      }
    }

    if (remaining_recv_q_length <= 2 && !iq_empty(&reg_q) && mem[iq_front(&reg_q)] == NULL) { /* :199-216 */
      int k = iq_pop(&reg_q);
      mem[k] = pool_get(&pool);
      if (!mem[k]) break;
      remaining_recv_q_length++;
      net_recv(w, r, from, mem[k], BYTES(k));
    }

    if (!iq_empty(&first_send_q)) {                                     /* :218-235 */
      int i = iq_pop(&first_send_q);
      mem[i] = pool_get(&pool);
      if (!mem[i]) break;
      memcpy(mem[i], R->sendbuf + BOFF(i), BYTES(i));
      iq_push(&wait_send_q, i);
    }

    if (!iq_empty(&wait_send_q)) {                                      /* :237-255 */
      int i = iq_pop(&wait_send_q);
      net_send(w, r, to, mem[i], BYTES(i), OFF(i));
      iq_push(&wait_send_completion_q, i);
    } else if (iq_empty(&first_send_q) && iq_empty(&wait_send_q) && !iq_empty(&buffering)) { /* :256-273 */
      while (!iq_empty(&buffering)) {
        int i = iq_pop(&buffering);
        net_send(w, r, to, mem[i], BYTES(i), OFF(i));
        iq_push(&wait_send_completion_q, i);
      }
    }

    while (net_send_poll(w, r, to)) {                                   /* :275-286 */
      int c = iq_pop(&wait_send_completion_q);
      pool_put(&pool, mem[c]);
      mem[c] = NULL;
    }
    sched_yield();
  }

  while (!iq_empty(&wait_send_completion_q) && !w->abort_flag && !pool.failed) { /* :290-299 */
    if (!net_send_wait(w, r, to)) break;
    int c = iq_pop(&wait_send_completion_q);
    pool_put(&pool, mem[c]);
    mem[c] = NULL;
  }

  if (pool.failed) R->rc = ORC_INTERNAL;
  R->pool_high_water = pool.high_water;
  R->pool_blocks = pool.n_blocks;
  R->slots_leaked = pool.held;
  iq_free(&reg_q); iq_free(&first_send_q); iq_free(&buffering);
  iq_free(&wait_send_q); iq_free(&wait_reduction_q); iq_free(&wait_send_completion_q);
  free(mem);
  pool_destroy(&pool);
  part_free(&P);
}

/* ------------------------------------------------------------------------ */
/* AllreduceRabenseifnerCuda<T>, allreduce_cuda_impl.h:326-717               */
/* ------------------------------------------------------------------------ */

static chunk_t mk_chunk(int range_id, int depth, int pair_rank, int reduce, int last) {
  chunk_t c = {range_id, depth, pair_rank, reduce, last};
  return c;
}

static void raben_gpu(rank_t* R) {
  world_t* w = R->w;
  const int N = w->n, r = R->rank;
  const size_t es = w->esize;

  memcpy(R->recvbuf, R->sendbuf, es * R->len);                          /* :332-333, before any check */
  if (N == 1) return;                                                   /* :335-340 */
  const int exp = orc_get_exp_of_two(N);                                /* :342 */
  if (exp == 0) { R->rc = ORC_NOT_SUPPORTED; return; }                 /* :345-351 */

  part_t P;
  R->rc = part_build(&P, R->len, es, N, R->env_chunk);                 /* :353-354 */
  if (R->rc) { part_free(&P); return; }
  const int chunks = P.n_ranges;

  pool_t pool;
  pool_init(&pool, R->pool_block, BYTES(0));                            /* :358-359 */
  char** mem = (char**)calloc((size_t)chunks, sizeof(char*));
  char* reduced_chunk = (char*)calloc((size_t)chunks, 1);               /* :362 */
  char* tmp_gpu_buffer = (char*)malloc(BYTES(0));                       /* :372-385: at least one chunk */

  cq recv_q = {0}, wait_recv_q = {0}, send_q = {0}, wait_send_q = {0};
  cq wait_send_copy_q = {0}, wait_reduction_q = {0}, first_send_q = {0}, buffering = {0};

  int start_rank = 0, end_rank = N;
  for (int step = 0; step < exp; step++) {                              /* :391-428 */
    int to = r ^ (1 << step);
    int ss, se, rs, re;
    if (r < to) { ss = start_rank; se = end_rank - (end_rank - start_rank) / 2; rs = se; re = end_rank; }
    else        { rs = start_rank; re = end_rank - (end_rank - start_rank) / 2; ss = re; se = end_rank; }
    for (int g = rs; g < re; g++)
      for (int c = P.first[g]; c < P.first[g] + P.count[g]; c++) cq_push(&recv_q, mk_chunk(c, step, to, 1, 0));
    for (int g = ss; g < se; g++)
      for (int c = P.first[g]; c < P.first[g] + P.count[g]; c++) {
        if (step == 0) cq_push(&first_send_q, mk_chunk(c, step, to, 0, 0));
        else           cq_push(&send_q, mk_chunk(c, step, to, 0, 0));
      }
    start_rank = rs; end_rank = re;
  }
  for (int step = 0; step < exp; step++) {                              /* :431-466 */
    int to = r ^ (1 << (exp - step - 1));
    int ss = start_rank, se = end_rank, rs, re;
    if (r > to) { rs = se; re = rs + end_rank - start_rank; }
    else        { re = ss; rs = re - (end_rank - start_rank); }
    for (int g = rs; g < re; g++)
      for (int c = P.first[g]; c < P.first[g] + P.count[g]; c++) cq_push(&recv_q, mk_chunk(c, step + exp, to, 0, 0));
    for (int g = ss; g < se; g++)
      for (int c = P.first[g]; c < P.first[g] + P.count[g]; c++)
        cq_push(&send_q, mk_chunk(c, step + exp, to, 1, step == exp - 1));
    start_rank = ss < rs ? ss : rs;
    end_rank = se > re ? se : re;
  }

  while (!cq_empty(&recv_q) || !cq_empty(&wait_recv_q) || !cq_empty(&send_q) || !cq_empty(&wait_send_q) ||
         !cq_empty(&wait_send_copy_q) || !cq_empty(&wait_reduction_q) || !cq_empty(&first_send_q) ||
         !cq_empty(&buffering)) {                                       /* :470-473 */
    if (world_dead(w) || pool.failed) break;

    while (cq_empty(&wait_reduction_q) && !cq_empty(&wait_recv_q) &&
           net_recv_poll(w, r, cq_front(&wait_recv_q).pair_rank)) {     /* :474-475 */
      chunk_t got = cq_pop(&wait_recv_q);
      int id = got.range_id;
      char* m = mem[id];
      if (got.reduce) {
        memcpy(tmp_gpu_buffer, m, BYTES(id));                           /* :503-504 */
        orc_reduce_inplace(w->dtype, R->recvbuf + BOFF(id), tmp_gpu_buffer, NEL(id)); /* :510-512 */
        memcpy(m, R->recvbuf + BOFF(id), BYTES(id));                    /* :515-516 */
        got.depth++;                                                    /* :518 */
        cq_push(&wait_reduction_q, got);
      } else {
        memcpy(R->recvbuf + BOFF(id), m, BYTES(id));                    /* :528-529 */
        reduced_chunk[id] = 1;
      }
    }

    if (!cq_empty(&wait_reduction_q)) {                                 /* :537-581 */
      chunk_t red = cq_pop(&wait_reduction_q);
      int id = red.range_id;
      if (!cq_empty(&send_q) && cq_front(&send_q).range_id == id && cq_front(&send_q).depth == red.depth) {
        chunk_t s = cq_pop(&send_q);
        if (cq_empty(&first_send_q) && cq_empty(&wait_send_copy_q) && cq_empty(&buffering)) {
          net_send(w, r, s.pair_rank, mem[id], BYTES(id), OFF(id));
          cq_push(&wait_send_q, s);
        } else {
          cq_push(&buffering, s);
        }
        if (s.reduce) reduced_chunk[s.range_id] = 1;                    /* :572-575 */
      } else {
        pool_put(&pool, mem[id]);                                       /* :577-579 */
        mem[id] = NULL;
      }
    }

    if (cq_size(&wait_recv_q) <= 2 && !cq_empty(&recv_q) && mem[cq_front(&recv_q).range_id] == NULL) { /* :583-601 */
      chunk_t rr = cq_pop(&recv_q);
      mem[rr.range_id] = pool_get(&pool);
      if (!mem[rr.range_id]) break;
      net_recv(w, r, rr.pair_rank, mem[rr.range_id], BYTES(rr.range_id));
      cq_push(&wait_recv_q, rr);
    }

    while (cq_empty(&first_send_q) && cq_empty(&wait_send_copy_q) && cq_empty(&buffering) &&
           !cq_empty(&send_q) && reduced_chunk[cq_front(&send_q).range_id]) { /* :603-622 */
      chunk_t s = cq_pop(&send_q);
      net_send(w, r, s.pair_rank, mem[s.range_id], BYTES(s.range_id), OFF(s.range_id));
      cq_push(&wait_send_q, s);
    }

    if (!cq_empty(&first_send_q)) {                                     /* :624-642 */
      chunk_t s = cq_pop(&first_send_q);
      mem[s.range_id] = pool_get(&pool);
      if (!mem[s.range_id]) break;
      memcpy(mem[s.range_id], R->sendbuf + BOFF(s.range_id), BYTES(s.range_id));
      cq_push(&wait_send_copy_q, s);
    }

    if (!cq_empty(&wait_send_copy_q)) {                                 /* :644-664 */
      chunk_t s = cq_pop(&wait_send_copy_q);
      net_send(w, r, s.pair_rank, mem[s.range_id], BYTES(s.range_id), OFF(s.range_id));
      cq_push(&wait_send_q, s);
    }

    while (cq_empty(&first_send_q) && cq_empty(&wait_send_copy_q) && !cq_empty(&buffering)) { /* :666-684 */
      chunk_t s = cq_pop(&buffering);
      net_send(w, r, s.pair_rank, mem[s.range_id], BYTES(s.range_id), OFF(s.range_id));
      cq_push(&wait_send_q, s);
    }

    while (!cq_empty(&wait_send_q) && net_send_poll(w, r, cq_front(&wait_send_q).pair_rank)) { /* :686-705 */
      chunk_t s = cq_pop(&wait_send_q);
      if (s.reduce && !s.last) {
        /* slot kept: the same data is sent again at the next doubling step */
      } else {
        pool_put(&pool, mem[s.range_id]);
        mem[s.range_id] = NULL;
      }
    }
    sched_yield();
  }

  if (pool.failed) R->rc = ORC_INTERNAL;
  R->pool_high_water = pool.high_water;
  for (int i = 0; i < chunks; i++)                                      /* :709-715 */
    if (mem[i]) { pool_put(&pool, mem[i]); mem[i] = NULL; }
  R->pool_blocks = pool.n_blocks;
  R->slots_leaked = pool.held;

  cq_free(&recv_q); cq_free(&wait_recv_q); cq_free(&send_q); cq_free(&wait_send_q);
  cq_free(&wait_send_copy_q); cq_free(&wait_reduction_q); cq_free(&first_send_q); cq_free(&buffering);
  free(mem); free(reduced_chunk); free(tmp_gpu_buffer);
  pool_destroy(&pool);
  part_free(&P);
}

/* ------------------------------------------------------------------------ */
/* driver                                                                   */
/* ------------------------------------------------------------------------ */

static world_t* g_last_world = NULL;

static void world_free(world_t* w) {
  if (!w) return;
  for (int i = 0; i < w->n * w->n; i++) {
    channel_t* c = &w->ch[i];
    pthread_mutex_destroy(&c->mu);
    pq_free(&c->sends); pq_free(&c->recvs);
    free(c->log_off); free(c->log_n);
  }
  free(w->ch);
  free(w);
}

static void* rank_main(void* arg) {
  rank_t* R = (rank_t*)arg;
  switch (R->algo) {
    case ORC_RING_CPU: ring_cpu(R); break;
    case ORC_RABEN_CPU: raben_cpu(R); break;
    case ORC_RING_GPU: ring_gpu(R); break;
    case ORC_RABEN_GPU: raben_gpu(R); break;
    default: R->rc = ORC_INVALID_ARGUMENT; break;
  }
  /* the reference exits the process on error; here the other ranks must not
   * wait for a peer that has left */
  if (R->rc) R->w->abort_flag = 1;
  return NULL;
}

int orc_allreduce(int algo, int dtype, int world_size, const void* const* sendbufs,
                  void* const* recvbufs, size_t len_elements, const char* env_chunksize,
                  size_t pool_block_bytes, orc_stats* stats) {
  if (world_size < 1 || orc_dtype_size(dtype) == 0) return ORC_INVALID_ARGUMENT;
  world_free(g_last_world);
  g_last_world = NULL;

  world_t* w = (world_t*)calloc(1, sizeof(world_t));
  w->n = world_size;
  w->dtype = dtype;
  w->esize = orc_dtype_size(dtype);
  w->ch = (channel_t*)calloc((size_t)world_size * (size_t)world_size, sizeof(channel_t));
  for (int i = 0; i < world_size * world_size; i++) pthread_mutex_init(&w->ch[i].mu, NULL);
  const char* dl = getenv("IBCOMM_ORACLE_DEADLINE_S");
  w->deadline = now_s() + (dl ? atof(dl) : 600.0);

  rank_t* R = (rank_t*)calloc((size_t)world_size, sizeof(rank_t));
  pthread_t* th = (pthread_t*)calloc((size_t)world_size, sizeof(pthread_t));
  for (int r = 0; r < world_size; r++) {
    R[r].w = w; R[r].rank = r; R[r].algo = algo;
    R[r].sendbuf = (const char*)sendbufs[r];
    R[r].recvbuf = (char*)recvbufs[r];
    R[r].len = len_elements;
    R[r].env_chunk = env_chunksize;
    R[r].pool_block = pool_block_bytes ? pool_block_bytes : (size_t)64 * 1024 * 1024; /* memory_pool.h:83 */
  }
  for (int r = 0; r < world_size; r++) pthread_create(&th[r], NULL, rank_main, &R[r]);
  for (int r = 0; r < world_size; r++) pthread_join(th[r], NULL);

  int rc = ORC_OK;
  orc_stats st = {0, 0, 0, 0};
  for (int r = 0; r < world_size; r++) {
    if (R[r].rc && !rc) rc = R[r].rc;
    if (R[r].pool_high_water > st.pool_slots_high_water) st.pool_slots_high_water = R[r].pool_high_water;
    if (R[r].pool_blocks > st.pool_blocks) st.pool_blocks = R[r].pool_blocks;
    st.slots_leaked += R[r].slots_leaked;
  }
  st.messages = w->messages;
  if (!rc && w->abort_flag) rc = ORC_INTERNAL;
  if (stats) *stats = st;
  free(R); free(th);
  g_last_world = w;
  return rc;
}

long orc_wire_count(int src, int dst) {
  world_t* w = g_last_world;
  if (!w || src < 0 || dst < 0 || src >= w->n || dst >= w->n) return -1;
  return w->ch[src * w->n + dst].log_count;
}

int orc_wire_get(int src, int dst, long k, size_t* offset_elements, size_t* n_elements) {
  world_t* w = g_last_world;
  if (!w || src < 0 || dst < 0 || src >= w->n || dst >= w->n) return ORC_INVALID_ARGUMENT;
  channel_t* c = &w->ch[src * w->n + dst];
  if (k < 0 || k >= c->log_count) return ORC_INVALID_ARGUMENT;
  *offset_elements = c->log_off[k];
  *n_elements = c->log_n[k];
  return ORC_OK;
}

/* ------------------------------------------------------------------------ */
/* closed forms                                                             */
/* ------------------------------------------------------------------------ */

int orc_closed_form_ring(int dtype, int world_size, const void* const* sendbufs, void* out,
                         size_t len_elements, const char* env_chunksize) {
  const size_t es = orc_dtype_size(dtype);
  if (!es || world_size < 1) return ORC_INVALID_ARGUMENT;
  const int N = world_size;
  if (N == 1) { memcpy(out, sendbufs[0], es * len_elements); return ORC_OK; }
  part_t P;
  int rc = part_build(&P, len_elements, es, N, env_chunksize);
  if (rc) { part_free(&P); return rc; }
  for (int g = 0; g < N; g++) {
    for (int c = P.first[g]; c < P.first[g] + P.count[g]; c++) {
      char* o = (char*)out + BOFF(c);
      memcpy(o, (const char*)sendbufs[g] + BOFF(c), BYTES(c));
      for (int j = 1; j < N; j++)
        orc_reduce_inplace(dtype, o, (const char*)sendbufs[(g + j) % N] + BOFF(c), NEL(c));
    }
  }
  part_free(&P);
  return ORC_OK;
}

int orc_closed_form_tree(int dtype, int world_size, const void* const* sendbufs, void* out,
                         size_t len_elements) {
  const size_t es = orc_dtype_size(dtype);
  if (!es || world_size < 1) return ORC_INVALID_ARGUMENT;
  const int N = world_size;
  if (N == 1) { memcpy(out, sendbufs[0], es * len_elements); return ORC_OK; }
  if (orc_get_exp_of_two(N) == 0) return ORC_NOT_SUPPORTED;
  const size_t B = 16384; /* elements per block, keeps the N partial rows in cache */
  char* rows = (char*)malloc((size_t)N * B * es);
  for (size_t base = 0; base < len_elements; base += B) {
    size_t n = len_elements - base < B ? len_elements - base : B;
    for (int r = 0; r < N; r++) memcpy(rows + (size_t)r * B * es, (const char*)sendbufs[r] + base * es, n * es);
    for (int stride = 1; stride < N; stride <<= 1)
      for (int r = 0; r < N; r += 2 * stride)
        orc_reduce_inplace(dtype, rows + (size_t)r * B * es, rows + (size_t)(r + stride) * B * es, n);
    memcpy((char*)out + base * es, rows, n * es);
  }
  free(rows);
  return ORC_OK;
}

/* ------------------------------------------------------------------------ */
/* CPU baseline helper                                                      */
/* ------------------------------------------------------------------------ */

double orc_time_reduce_f32(size_t n, int reps) {
  float* a = (float*)malloc(n * sizeof(float));
  float* b = (float*)malloc(n * sizeof(float));
  if (!a || !b) { free(a); free(b); return -1.0; }
  for (size_t i = 0; i < n; i++) { a[i] = 0.0f; b[i] = (float)(i & 1023) * 0.25f; }
  double best = 1e30;
  for (int k = 0; k < reps; k++) {
    double t0 = now_s();
    reduce_f32(a, b, n);
    double t1 = now_s();
    if (t1 - t0 < best) best = t1 - t0;
  }
  volatile float sink = a[n / 2];
  (void)sink;
  free(a); free(b);
  return best;
}
