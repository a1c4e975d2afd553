/*
 * tp_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of what pytorch/tensorpipe's device channels compute for a
 * message: the payload-byte semantics of cuda_xth, cuda_ipc and cuda_basic,
 * their chunking arithmetic and their slot allocator. It exists so that the
 * HIP channels can be checked against the reference's behaviour on the same
 * inputs. Only tests, the smoke check and the CPU-baseline leg of the bench
 * may load it; no product code path may call into it.
 *
 * How each function is pinned (none is "parity unpinned"):
 *  - The three copy restatements are the identity on bytes by construction of
 *    the reference (every copy site is a memcpy/cudaMemcpyAsync of `length`
 *    bytes); they are checked against the reference's own test vectors
 *    (256 B iota, 100 x 256 KiB of i%256, 0x42 fills, the base+128 offset
 *    send, zero-length and 1,0,1 sequences) and against plain memcmp with the
 *    input plus untouched guard bands.
 *  - Chunk arithmetic is checked by brute force over lengths around every
 *    multiple of the slot size and by the invariants sum(chunks) == length,
 *    every chunk but the last == slot.
 *  - The allocator simulation is checked against a hand-worked trace
 *    (lowest free slot first, FIFO waiters, close fails waiters).
 *
 * Paths are relative to the root of pytorch/tensorpipe.
 */
#ifndef TP_ORACLE_H_
#define TP_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tp_oracle_copy_desc {
  const void* src;
  void* dst;
  uint64_t bytes;
} tp_oracle_copy_desc;

/* cuda_xth: one cudaMemcpyAsync(dst, src, length) per tensor,
 * tensorpipe/channel/cuda_xth/channel_impl.cc:66-77; zero length is a no-op,
 * :122-126. A message is a sequence of such copies in order,
 * tensorpipe/core/pipe_impl.cc:471-511. */
void tp_oracle_xth_message(const tp_oracle_copy_desc* table, uint32_t n);

/* ceilOfRatio(length, slot) chunks; chunk k has min(length - k*slot, slot)
 * bytes: tensorpipe/channel/cuda_ipc/channel_impl.cc:117-131 and
 * tensorpipe/channel/cuda_basic/channel_impl.cc:84-114. */
uint64_t tp_oracle_num_chunks(uint64_t length, uint64_t slot);
uint64_t tp_oracle_chunk_length(uint64_t length, uint64_t slot, uint64_t k);

/* cuda_ipc: every chunk is copied source -> outbox slot on the sender
 * (channel_impl.cc:238-252) and outbox slot -> target on the receiver
 * (:431-467). `outbox` is num_slots*slot bytes; with replies arriving in order
 * the allocator hands out the lowest free slot, and at most num_slots chunks
 * are in flight (tensorpipe/channel/cuda_ipc/constants.h:22-24: 4 x 8 MiB).
 * `in_flight` (1..num_slots) says how many chunks are staged before the oldest
 * one is drained, which exercises slot reuse. Returns chunks processed. */
uint64_t tp_oracle_ipc_tensor(const void* src, void* dst, uint64_t length, void* outbox,
                              uint64_t slot, uint32_t num_slots, uint32_t in_flight);

/* cuda_basic: per chunk GPU -> pinned send slot (channel_impl.cc:172-179,
 * 58-71), pinned slot -> inner CPU channel -> pinned recv slot (:209-214 and
 * :455-470), pinned recv slot -> GPU (:472-498).
 * tensorpipe/channel/cuda_basic/constants.h:22-24: 16 x 1 MiB per ring. The
 * inner CPU channel is the byte stream of tp_oracle_basic_stream. */
uint64_t tp_oracle_staged_tensor(const void* src, void* dst, uint64_t length, void* send_ring,
                                 void* recv_ring, uint64_t slot, uint32_t num_slots);

/* basic channel over a connection: the tensor's bytes are written to and read
 * from the connection unchanged, tensorpipe/channel/basic/channel_impl.cc:85-97,
 * 152-169. Modelled as a bounded byte ring of `ring_bytes` (power of two)
 * moved in pieces that fit, as the shm transport does
 * (tensorpipe/common/ringbuffer_read_write_ops.h:236-283). */
void tp_oracle_basic_stream(const void* src, void* dst, uint64_t length, void* ring,
                            uint64_t ring_bytes);

/* Benchmark fill pattern data[i] = (i >> 8) ^ (i & 0xff),
 * tensorpipe/benchmark/benchmark_pipe.cc:144-151. */
void tp_oracle_bench_pattern(uint8_t* data, uint64_t n);

/* percentile(f) = sorted[floor(f * n)],
 * tensorpipe/benchmark/measurements.h:51-53. Sorts in place. */
double tp_oracle_percentile(double* samples, uint64_t n, double f);

/* Slot allocator simulation, tensorpipe/common/allocator.cc:26-79.
 * Events are executed in order; op 'a' = alloc request (id = arg), 'r' =
 * release of slot arg, 'c' = close. For every alloc request that gets served,
 * appends (request id, slot index) to out; a request failed by close appends
 * (id, -1). Returns the number of pairs written (each pair is two ints). */
typedef struct tp_oracle_alloc_event {
  char op;
  int32_t arg;
} tp_oracle_alloc_event;
uint32_t tp_oracle_allocator_trace(uint32_t num_slots, const tp_oracle_alloc_event* events,
                                   uint32_t num_events, int32_t* out, uint32_t out_cap);

#ifdef __cplusplus
}
#endif
#endif /* TP_ORACLE_H_ */
