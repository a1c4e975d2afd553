/*
 * cpu_shm_basic.c -- TEST / BASELINE INFRASTRUCTURE ONLY (never on a product
 * path). CPU port of the reference's shm transport + basic channel ping-pong,
 * i.e. what `benchmark_pipe --transport shm --channel basic` times
 * (tensorpipe/benchmark/benchmark_pipe.cc:422-636) for CPU tensors. It is the
 * "port" CPU baseline that the bench reports beside the GPU figures.
 *
 * What is restated, and from where:
 *  - one single-producer single-consumer byte ring of 2 MiB per connection and
 *    direction (kBufferSize, tensorpipe/transport/shm/connection_impl.h:38),
 *    head/tail counters, producer copies in what fits, consumer copies out
 *    (tensorpipe/common/ringbuffer_role.h:26-283);
 *  - every message is a uint32 length followed by the bytes, streamed through
 *    the ring in pieces (tensorpipe/common/ringbuffer_read_write_ops.h:138-283);
 *  - each process runs ONE busy-polling reactor thread that does all ring
 *    traffic of that process (tensorpipe/transport/shm/reactor.cc:111-135);
 *  - a pipe message with one tensor and one payload is, on the wire
 *    (tensorpipe/core/pipe_impl.cc:536-581,728-748,795-825): descriptor and
 *    payload on the pipe's connection, a descriptor reply back (the benchmark
 *    sets no target device), then the tensor bytes on the basic channel's own
 *    connection (tensorpipe/channel/basic/channel_impl.cc:85-97,152-169);
 *  - the initiator times write -> echoed read per round trip and percentiles
 *    are sorted[floor(f*n)] (tensorpipe/benchmark/measurements.h:51-53).
 *
 * What is left out: the deferred-function queues, locks, std::function and
 * shared_ptr traffic, nop (de)serialisation and the reactor token ring of the
 * real thing. The port therefore runs FASTER than the reference would on the
 * same cores; read it as a lower bound on the reference's latency and an upper
 * bound on its throughput.
 *
 * Pinned by: the payload bytes received are compared with the bytes sent on
 * every round trip (identity), and the ring arithmetic is the same as
 * tp_oracle_basic_stream, which tests/test_oracle.py checks against wrap-around
 * cases.
 *
 * Usage: cpu_shm_basic <tensor_bytes> <payload_bytes> <warmup> <iters>
 * Prints one JSON line. Uses 2 cores (one busy thread per process).
 */
#define _GNU_SOURCE
#include <stdatomic.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/wait.h>
#include <time.h>
#include <unistd.h>

#define RING_BYTES (2u * 1024u * 1024u)

typedef struct {
  _Alignas(64) _Atomic uint64_t head;
  _Alignas(64) _Atomic uint64_t tail;
  _Alignas(64) uint8_t data[RING_BYTES];
} ring_t;

typedef struct {
  ring_t to_server;
  ring_t to_client;
} conn_t;

typedef struct {
  conn_t pipe; /* descriptors, payloads, descriptor replies */
  conn_t chan; /* basic channel: tensor bytes */
  _Atomic int failed;
} shared_t;

static inline void cpu_relax(void) {
#if defined(__x86_64__)
  __builtin_ia32_pause();
#endif
}

static void ring_write(ring_t* r, const void* src, uint64_t n) {
  const uint8_t* s = (const uint8_t*)src;
  while (n > 0) {
    uint64_t head = atomic_load_explicit(&r->head, memory_order_relaxed);
    uint64_t tail = atomic_load_explicit(&r->tail, memory_order_acquire);
    uint64_t space = RING_BYTES - (head - tail);
    if (space == 0) {
      cpu_relax();
      continue;
    }
    uint64_t put = n < space ? n : space;
    uint64_t pos = head & (RING_BYTES - 1);
    uint64_t first = put < RING_BYTES - pos ? put : RING_BYTES - pos;
    memcpy(r->data + pos, s, first);
    if (put > first) {
      memcpy(r->data, s + first, put - first);
    }
    atomic_store_explicit(&r->head, head + put, memory_order_release);
    s += put;
    n -= put;
  }
}

static void ring_read(ring_t* r, void* dst, uint64_t n) {
  uint8_t* d = (uint8_t*)dst;
  while (n > 0) {
    uint64_t tail = atomic_load_explicit(&r->tail, memory_order_relaxed);
    uint64_t head = atomic_load_explicit(&r->head, memory_order_acquire);
    uint64_t avail = head - tail;
    if (avail == 0) {
      cpu_relax();
      continue;
    }
    uint64_t get = n < avail ? n : avail;
    uint64_t pos = tail & (RING_BYTES - 1);
    uint64_t first = get < RING_BYTES - pos ? get : RING_BYTES - pos;
    memcpy(d, r->data + pos, first);
    if (get > first) {
      memcpy(d + first, r->data, get - first);
    }
    atomic_store_explicit(&r->tail, tail + get, memory_order_release);
    d += get;
    n -= get;
  }
}

static void msg_write(ring_t* r, const void* p, uint32_t len) {
  ring_write(r, &len, sizeof(len));
  ring_write(r, p, len);
}

/* Reads a message that must have exactly `len` bytes. */
static int msg_read(ring_t* r, void* p, uint32_t len) {
  uint32_t got = 0;
  ring_read(r, &got, sizeof(got));
  if (got != len) {
    return -1;
  }
  ring_read(r, p, len);
  return 0;
}

/* Stand-ins for the serialised Descriptor and DescriptorReply: sizes are what
 * nop produces for one payload + one tensor with short metadata strings. */
typedef struct {
  uint8_t bytes[96];
} descriptor_t;
typedef struct {
  uint8_t bytes[24];
} reply_t;

static int send_message(ring_t* pipe_out, ring_t* pipe_in, ring_t* chan_out, const void* payload,
                        uint32_t payload_len, const void* tensor, uint64_t tensor_len) {
  descriptor_t d;
  memset(&d, 0, sizeof(d));
  memcpy(d.bytes, &tensor_len, 8);
  memcpy(d.bytes + 8, &payload_len, 4);
  msg_write(pipe_out, &d, sizeof(d));
  if (payload_len > 0) {
    msg_write(pipe_out, payload, payload_len);
  }
  reply_t rep;
  if (msg_read(pipe_in, &rep, sizeof(rep)) != 0) {
    return -1;
  }
  /* basic channel: the tensor is one message on the channel's connection;
   * lengths beyond 4 GiB are out of scope for this port */
  msg_write(chan_out, tensor, (uint32_t)tensor_len);
  return 0;
}

static int recv_message(ring_t* pipe_in, ring_t* pipe_out, ring_t* chan_in, void* payload,
                        uint32_t payload_len, void* tensor, uint64_t tensor_len) {
  descriptor_t d;
  if (msg_read(pipe_in, &d, sizeof(d)) != 0) {
    return -1;
  }
  uint64_t tl;
  memcpy(&tl, d.bytes, 8);
  if (tl != tensor_len) {
    return -1;
  }
  if (payload_len > 0 && msg_read(pipe_in, payload, payload_len) != 0) {
    return -1;
  }
  reply_t rep;
  memset(&rep, 0, sizeof(rep));
  msg_write(pipe_out, &rep, sizeof(rep));
  return msg_read(chan_in, tensor, (uint32_t)tensor_len);
}

static double now_us(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return ts.tv_sec * 1e6 + ts.tv_nsec * 1e-3;
}

static int cmp_double(const void* a, const void* b) {
  double x = *(const double*)a, y = *(const double*)b;
  return (x > y) - (x < y);
}

int main(int argc, char** argv) {
  if (argc < 5) {
    fprintf(stderr, "usage: %s tensor_bytes payload_bytes warmup iters\n", argv[0]);
    return 2;
  }
  const uint64_t tensor_len = strtoull(argv[1], NULL, 10);
  const uint32_t payload_len = (uint32_t)strtoul(argv[2], NULL, 10);
  const int warmup = atoi(argv[3]);
  const int iters = atoi(argv[4]);
  if (tensor_len == 0 || tensor_len >= (1ull << 32) || iters <= 0) {
    fprintf(stderr, "tensor_bytes must be in [1, 4 GiB), iters > 0\n");
    return 2;
  }

  shared_t* sh = (shared_t*)mmap(NULL, sizeof(shared_t), PROT_READ | PROT_WRITE,
                                 MAP_SHARED | MAP_ANONYMOUS, -1, 0);
  if (sh == MAP_FAILED) {
    perror("mmap");
    return 1;
  }
  memset(sh, 0, sizeof(*sh));

  uint8_t* tensor = (uint8_t*)malloc(tensor_len);
  uint8_t* back = (uint8_t*)malloc(tensor_len);
  uint8_t* payload = (uint8_t*)malloc(payload_len ? payload_len : 1);
  uint8_t* payload_back = (uint8_t*)malloc(payload_len ? payload_len : 1);
  /* benchmark fill pattern, tensorpipe/benchmark/benchmark_pipe.cc:144-151 */
  for (uint64_t i = 0; i < tensor_len; ++i) {
    tensor[i] = (uint8_t)((i >> 8) ^ (i & 0xff));
  }
  for (uint32_t i = 0; i < payload_len; ++i) {
    payload[i] = (uint8_t)((i >> 8) ^ (i & 0xff));
  }
  memset(back, 0, tensor_len);

  pid_t pid = fork();
  if (pid < 0) {
    perror("fork");
    return 1;
  }
  if (pid == 0) {
    /* server: echo */
    for (int it = 0; it < warmup + iters; ++it) {
      if (recv_message(&sh->pipe.to_server, &sh->pipe.to_client, &sh->chan.to_server, payload_back,
                       payload_len, back, tensor_len) != 0 ||
          send_message(&sh->pipe.to_client, &sh->pipe.to_server, &sh->chan.to_client, payload_back,
                       payload_len, back, tensor_len) != 0) {
        atomic_store(&sh->failed, 1);
        _exit(1);
      }
    }
    _exit(0);
  }

  double* samples = (double*)malloc(sizeof(double) * iters);
  double begin = 0;
  int mismatches = 0;
  for (int it = 0; it < warmup + iters; ++it) {
    if (it == warmup) {
      begin = now_us();
    }
    double t0 = now_us();
    if (send_message(&sh->pipe.to_server, &sh->pipe.to_client, &sh->chan.to_server, payload,
                     payload_len, tensor, tensor_len) != 0 ||
        recv_message(&sh->pipe.to_client, &sh->pipe.to_server, &sh->chan.to_client, payload_back,
                     payload_len, back, tensor_len) != 0) {
      fprintf(stderr, "protocol error\n");
      return 1;
    }
    double t1 = now_us();
    if (it >= warmup) {
      samples[it - warmup] = t1 - t0;
    }
    if (memcmp(back, tensor, tensor_len) != 0 || memcmp(payload_back, payload, payload_len) != 0) {
      ++mismatches;
    }
  }
  double total_us = now_us() - begin;
  int st = 0;
  waitpid(pid, &st, 0);
  qsort(samples, iters, sizeof(double), cmp_double);
  double p50 = samples[(size_t)(0.5 * iters)];
  double p95 = samples[(size_t)(0.95 * iters) < (size_t)iters ? (size_t)(0.95 * iters) : (size_t)iters - 1];
  /* each round trip carries the tensor once in each direction */
  double gbps = 2.0 * (double)tensor_len * iters / (total_us * 1e-6) / 1e9;
  printf("{\"kind\": \"port\", \"tensor_bytes\": %llu, \"payload_bytes\": %u, \"iters\": %d, "
         "\"rtt_p50_us\": %.3f, \"rtt_p95_us\": %.3f, \"rtt_min_us\": %.3f, \"payload_GBps\": %.4f, "
         "\"mismatches\": %d, \"cores\": 2, \"child_status\": %d}\n",
         (unsigned long long)tensor_len, payload_len, iters, p50, p95, samples[0], gbps, mismatches,
         WEXITSTATUS(st));
  return mismatches == 0 && WEXITSTATUS(st) == 0 ? 0 : 1;
}
