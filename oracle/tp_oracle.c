/*
 * tp_oracle.c -- TEST INFRASTRUCTURE ONLY. See tp_oracle.h for what this
 * restates, which reference lines each function follows and how it is pinned.
 */
#include "tp_oracle.h"

#include <stdlib.h>
#include <string.h>

void tp_oracle_xth_message(const tp_oracle_copy_desc* table, uint32_t n) {
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].bytes == 0) {
      continue; /* zero length: callback only, nothing moves */
    }
    memcpy(table[i].dst, table[i].src, table[i].bytes);
  }
}

uint64_t tp_oracle_num_chunks(uint64_t length, uint64_t slot) {
  return (length + slot - 1) / slot;
}

uint64_t tp_oracle_chunk_length(uint64_t length, uint64_t slot, uint64_t k) {
  uint64_t offset = k * slot;
  uint64_t rest = length - offset;
  return rest < slot ? rest : slot;
}

uint64_t tp_oracle_ipc_tensor(const void* src, void* dst, uint64_t length, void* outbox,
                              uint64_t slot, uint32_t num_slots, uint32_t in_flight) {
  if (length == 0) {
    return 0;
  }
  if (in_flight < 1) {
    in_flight = 1;
  }
  if (in_flight > num_slots) {
    in_flight = num_slots;
  }
  const uint8_t* s = (const uint8_t*)src;
  uint8_t* d = (uint8_t*)dst;
  uint8_t* box = (uint8_t*)outbox;
  const uint64_t chunks = tp_oracle_num_chunks(length, slot);
  /* slot_of[c % in_flight] remembers which slot chunk c sits in. */
  int used[64];
  uint32_t slot_of[64];
  memset(used, 0, sizeof(used));
  uint64_t staged = 0, drained = 0;
  while (drained < chunks) {
    /* sender side: stage while a slot is free and the window allows it */
    while (staged < chunks && staged - drained < in_flight) {
      uint32_t sl = 0;
      while (used[sl]) {
        ++sl; /* lowest free slot first */
      }
      used[sl] = 1;
      slot_of[staged % in_flight] = sl;
      memcpy(box + (uint64_t)sl * slot, s + staged * slot,
             tp_oracle_chunk_length(length, slot, staged));
      ++staged;
    }
    /* receiver side: drain the oldest chunk, reply frees its slot */
    uint32_t sl = slot_of[drained % in_flight];
    memcpy(d + drained * slot, box + (uint64_t)sl * slot,
           tp_oracle_chunk_length(length, slot, drained));
    used[sl] = 0;
    ++drained;
  }
  return chunks;
}

void tp_oracle_basic_stream(const void* src, void* dst, uint64_t length, void* ring,
                            uint64_t ring_bytes) {
  const uint8_t* s = (const uint8_t*)src;
  uint8_t* d = (uint8_t*)dst;
  uint8_t* r = (uint8_t*)ring;
  uint64_t head = 0; /* bytes ever written */
  uint64_t tail = 0; /* bytes ever read */
  const uint64_t mask = ring_bytes - 1;
  while (tail < length) {
    /* producer: as much as fits, possibly in two pieces around the wrap */
    uint64_t space = ring_bytes - (head - tail);
    uint64_t put = length - head < space ? length - head : space;
    while (put > 0) {
      uint64_t pos = head & mask;
      uint64_t piece = ring_bytes - pos < put ? ring_bytes - pos : put;
      memcpy(r + pos, s + head, piece);
      head += piece;
      put -= piece;
    }
    /* consumer: everything available */
    uint64_t get = head - tail;
    while (get > 0) {
      uint64_t pos = tail & mask;
      uint64_t piece = ring_bytes - pos < get ? ring_bytes - pos : get;
      memcpy(d + tail, r + pos, piece);
      tail += piece;
      get -= piece;
    }
  }
}

uint64_t tp_oracle_staged_tensor(const void* src, void* dst, uint64_t length, void* send_ring,
                                 void* recv_ring, uint64_t slot, uint32_t num_slots) {
  if (length == 0) {
    return 0;
  }
  const uint8_t* s = (const uint8_t*)src;
  uint8_t* d = (uint8_t*)dst;
  uint8_t* sr = (uint8_t*)send_ring;
  uint8_t* rr = (uint8_t*)recv_ring;
  const uint64_t chunks = tp_oracle_num_chunks(length, slot);
  /* 2 MiB byte ring standing in for the shm connection's inbox. */
  const uint64_t ring_bytes = 2u * 1024u * 1024u;
  uint8_t* ring = (uint8_t*)malloc(ring_bytes);
  for (uint64_t k = 0; k < chunks; ++k) {
    const uint64_t len = tp_oracle_chunk_length(length, slot, k);
    /* Slots are released as soon as the chunk moved on, so with in-order
     * completion the lowest free slot cycles through the ring only when
     * several chunks are in flight; model a full window to exercise every
     * slot. */
    uint8_t* sslot = sr + (k % num_slots) * slot;
    uint8_t* rslot = rr + (k % num_slots) * slot;
    memcpy(sslot, s + k * slot, len);                        /* D2H */
    tp_oracle_basic_stream(sslot, rslot, len, ring, ring_bytes); /* inner CPU channel */
    memcpy(d + k * slot, rslot, len);                        /* H2D */
  }
  free(ring);
  return chunks;
}

void tp_oracle_bench_pattern(uint8_t* data, uint64_t n) {
  for (uint64_t i = 0; i < n; ++i) {
    data[i] = (uint8_t)((i >> 8) ^ (i & 0xff));
  }
}

static int cmp_double(const void* a, const void* b) {
  double x = *(const double*)a, y = *(const double*)b;
  return (x > y) - (x < y);
}

double tp_oracle_percentile(double* samples, uint64_t n, double f) {
  qsort(samples, n, sizeof(double), cmp_double);
  uint64_t idx = (uint64_t)(f * (double)n);
  if (idx >= n) {
    idx = n - 1;
  }
  return samples[idx];
}

uint32_t tp_oracle_allocator_trace(uint32_t num_slots, const tp_oracle_alloc_event* events,
                                   uint32_t num_events, int32_t* out, uint32_t out_cap) {
  int* avail = (int*)malloc(sizeof(int) * num_slots);
  int32_t* pending = (int32_t*)malloc(sizeof(int32_t) * (num_events + 1));
  uint32_t phead = 0, ptail = 0, written = 0;
  int closed = 0;
  for (uint32_t i = 0; i < num_slots; ++i) {
    avail[i] = 1;
  }
  for (uint32_t e = 0; e < num_events; ++e) {
    if (events[e].op == 'a') {
      pending[ptail++] = events[e].arg;
    } else if (events[e].op == 'r') {
      avail[events[e].arg] = 1;
    } else if (events[e].op == 'c') {
      closed = 1;
    }
    /* processAllocations(): serve the queue front-first until no slot is free */
    while (phead < ptail) {
      int32_t got = -1;
      if (!closed) {
        for (uint32_t sidx = 0; sidx < num_slots; ++sidx) {
          if (avail[sidx]) {
            avail[sidx] = 0;
            got = (int32_t)sidx;
            break;
          }
        }
        if (got < 0) {
          break;
        }
      }
      if (written + 2 <= out_cap) {
        out[written] = pending[phead];
        out[written + 1] = got;
      }
      written += 2;
      ++phead;
    }
  }
  free(avail);
  free(pending);
  return written / 2;
}
