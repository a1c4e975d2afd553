/*
 * tphip.h -- C ABI of libtphip.so, the only library in this tree that includes
 * HIP headers. The host-side channels (hip_xth, hip_ipc, hip_basic) reach the
 * GPU exclusively through these entry points.
 *
 * Conventions: every function returns 0 on success or a positive hipError_t
 * value (negative values are errors detected by this library itself, see
 * tphip_strerror). No exceptions, no C++ types, no reliance on the caller's
 * current device: every call that needs a device takes its index explicitly,
 * makes it current for its own duration and puts the caller's device back.
 * Streams and events are passed as void* (hipStream_t / hipEvent_t values).
 * All functions are thread-safe.
 *
 * Each declaration names the reference interface it replaces; paths are
 * relative to the root of pytorch/tensorpipe.
 */
#ifndef TPHIP_H_
#define TPHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPHIP_IPC_HANDLE_BYTES 64
#define TPHIP_UUID_STRLEN 36 /* 8-4-4-4-12 hex digits, NUL not counted */

/* Errors raised by the library itself (all negative). */
#define TPHIP_ERR_INVALID_ARG (-1)
#define TPHIP_ERR_TOO_LARGE (-2)
/* (-3 is not in use) */
#define TPHIP_ERR_NO_DEVICE (-4)
#define TPHIP_ERR_CAPTURING (-5)
#define TPHIP_ERR_BUSY (-6)

/* One entry of the copy table: `bytes` bytes from `src` to `dst`. Any
 * alignment, any length (including 0). Ranges of different entries must not
 * overlap each other's destinations, and no src range may overlap a dst range.
 * Replaces the (dst, src, length) triple handed to cudaMemcpyAsync at
 * tensorpipe/channel/cuda_xth/channel_impl.cc:69-71,
 * tensorpipe/channel/cuda_ipc/channel_impl.cc:244-249,456-461 and
 * tensorpipe/channel/cuda_basic/channel_impl.cc:58-71. */
typedef struct tphip_copy_desc {
  const void* src;
  void* dst;
  uint64_t bytes;
} tphip_copy_desc;

/* Largest table accepted by one tphip_batched_copy call. */
#define TPHIP_MAX_BATCH 4096u

const char* tphip_strerror(int err);

/* ---- devices and pointers ------------------------------------------------ */

/* Number of visible GPUs. Replaces cudaGetDeviceCount as used at
 * tensorpipe/channel/cuda_xth/context_impl.cc:52-56. */
int tphip_device_count(int* count);

/* Device UUID as a 36-character string plus NUL. Replaces
 * getUuidOfDevice/getUuidsOfVisibleDevices, tensorpipe/common/cuda.h:293-321. */
int tphip_device_uuid(int dev, char out[TPHIP_UUID_STRLEN + 1]);

/* Device ordinal that owns `ptr`; *dev = -1 for host memory unknown to HIP.
 * *is_host is set to 1 for (pinned) host allocations. Replaces
 * cudaDeviceForPointer, tensorpipe/common/cuda.h:141-166. */
int tphip_device_for_ptr(const void* ptr, int* dev, int* is_host);

/* Base address and size of the allocation containing `ptr` (needed because an
 * IPC handle always refers to the allocation base; cf. the offset test at
 * tensorpipe/test/channel/channel_test_cuda.cc:96-139). */
int tphip_mem_base(const void* ptr, void** base, size_t* size);

/* Identifier of the allocation containing `ptr`, unique for the lifetime of
 * the process; lets a cache keyed on the base address notice that the address
 * was freed and handed out again. *id = 0 when the runtime cannot tell. */
int tphip_mem_buffer_id(const void* ptr, uint64_t* id);

/* ---- memory -------------------------------------------------------------- */

/* Device slab. Replaces makeCudaDeviceBuffer, tensorpipe/common/cuda.h:213-218. */
int tphip_malloc(int dev, size_t bytes, void** ptr);
int tphip_free(int dev, void* ptr);

/* Pinned host slab, mapped into the device address space and portable across
 * devices. *dev_ptr (may be NULL) receives the address kernels use for it.
 * Replaces makeCudaPinnedBuffer, tensorpipe/common/cuda.h:183-188. */
int tphip_host_alloc(int dev, size_t bytes, void** host_ptr, void** dev_ptr);
int tphip_host_free(void* host_ptr);

/* ---- streams and events -------------------------------------------------- */

int tphip_stream_create(int dev, void** stream);
int tphip_stream_destroy(int dev, void* stream);
int tphip_stream_sync(int dev, void* stream);
/* *done = 1 when everything enqueued on `stream` so far has finished. */
int tphip_stream_query(int dev, void* stream, int* done);

/* interprocess != 0 creates an event exportable with tphip_ipc_event_export.
 * Timing is always disabled. Replaces CudaEvent,
 * tensorpipe/common/cuda.h:49-139. */
int tphip_event_create(int dev, int interprocess, void** event);
/* Timing-enabled event (bench and tests only). */
int tphip_event_create_timed(int dev, void** event);
int tphip_event_destroy(int dev, void* event);
int tphip_event_record(int dev, void* event, void* stream);
int tphip_stream_wait_event(int dev, void* stream, void* event);
/* *done = 1 when all work captured by the last record has finished. */
int tphip_event_query(int dev, void* event, int* done);
int tphip_event_sync(int dev, void* event);
int tphip_event_elapsed_ms(void* start, void* stop, float* ms);

/* Run fn(arg, status) on a runtime thread once all work enqueued on `stream`
 * so far has completed. Replaces CudaLoop::addCallback,
 * tensorpipe/common/cuda_loop.cc:86-124. */
typedef void (*tphip_host_fn)(void* arg, int status);
int tphip_stream_on_complete(int dev, void* stream, tphip_host_fn fn, void* arg);

/* ---- inter-process handles ----------------------------------------------- */

/* `base` must be the base of a device allocation (see tphip_mem_base).
 * Replaces cudaIpcGetMemHandle / cudaIpcOpenMemHandle / cudaIpcCloseMemHandle,
 * tensorpipe/common/cuda.h:226-268. */
int tphip_ipc_mem_export(int dev, void* base, uint8_t out[TPHIP_IPC_HANDLE_BYTES]);
int tphip_ipc_mem_open(int dev, const uint8_t handle[TPHIP_IPC_HANDLE_BYTES], void** ptr);
int tphip_ipc_mem_close(int dev, void* ptr);

/* Replaces cudaIpcGetEventHandle / cudaIpcOpenEventHandle,
 * tensorpipe/common/cuda.h:88-93,119-124. */
int tphip_ipc_event_export(int dev, void* event, uint8_t out[TPHIP_IPC_HANDLE_BYTES]);
int tphip_ipc_event_open(int dev, const uint8_t handle[TPHIP_IPC_HANDLE_BYTES], void** event);

/* ---- data movement ------------------------------------------------------- */

/* The hot path. Enqueue on `stream` ONE copy kernel that performs every copy
 * of `table[0..n)`; `table` is host memory and may be reused as soon as the
 * call returns. Tables of up to 256 entries travel in the kernel arguments (one
 * launch in all); larger ones are written to a pinned plan ring and moved to
 * device memory by a small staging kernel enqueued ahead of the copy kernel. Any mix of device, mapped-pinned-host and peer-mapped (IPC)
 * addresses is accepted as long as the device can address them. n == 0 or an
 * all-empty table enqueues nothing. n > TPHIP_MAX_BATCH returns
 * TPHIP_ERR_TOO_LARGE. A call whose plan travels in the kernel arguments (up
 * to 256 non-empty entries; tphip_copy always) may be captured into a HIP
 * graph: every replay copies between the same addresses. A larger table on a
 * capturing stream returns TPHIP_ERR_CAPTURING and enqueues nothing, because
 * the plan ring is rewritten by later calls. Replaces one cudaMemcpyAsync per tensor at the three
 * call sites listed for tphip_copy_desc. */
int tphip_batched_copy(int dev, const tphip_copy_desc* table, uint32_t n, void* stream);

/* tphip_batched_copy followed by tphip_event_record(event, stream), at lower
 * cost: the event becomes the completion signal of the call's last copy
 * kernel instead of a marker of its own behind it (about 2.5 us sooner seen
 * by a polling host, and no second submission). Where that is not possible
 * (nothing to enqueue, launch profiling on) the event is recorded plainly, so
 * after a successful call `event` always covers everything the call enqueued
 * and all earlier work of `stream`. Not for a stream that is being captured
 * into a graph (an event has no meaning there). `unroll`, `blocks` and `nontemporal` as
 * for tphip_batched_copy_tuned; 0, 0 and -1 select the defaults. The pair it
 * replaces: cudaMemcpyAsync +
 * cudaEventRecord at tensorpipe/channel/cuda_xth/channel_impl.cc:69-74,
 * tensorpipe/channel/cuda_ipc/channel_impl.cc:244-252,456-467. */
int tphip_batched_copy_signal(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                              void* event, int unroll, uint32_t blocks, int nontemporal);

/* tphip_batched_copy for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no
 * counterpart in the reference. tphip_batched_copy keeps the plans of larger
 * tables in rings of pinned and device memory that it allocates on first use;
 * this variant calls no hipMalloc, hipHostMalloc, hipFree or other allocating
 * routine, ever: its plan is written, by small kernels that carry it in their
 * arguments, into a device array that is part of the library image
 * (45 KiB per GPU the library runs on, held until the process ends), and the
 * same table kernel then reads it from there. Same table semantics and results
 * as tphip_batched_copy. Limits: n <= TPHIP_NOALLOC_MAX_BATCH, and the table's
 * 16-byte vectors must fit one launch (just under 64 GiB); beyond either the
 * call returns TPHIP_ERR_TOO_LARGE and enqueues nothing. All calls on one GPU
 * share that GPU's array: calls on one stream are ordered by the stream, calls
 * that may overlap on different streams of one GPU race and must be ordered
 * by the caller. Under capture every replay rewrites the array with the
 * captured plan before copying, so the same rule holds between a replay and
 * any other call. */
#define TPHIP_NOALLOC_MAX_BATCH 1024u
int tphip_batched_copy_noalloc(int dev, const tphip_copy_desc* table, uint32_t n, void* stream);

/* ---- signal words and the resident copy agent ------------------------------ */

/* Raises the 64-bit word at `word` (an address kernels can write: device
 * memory, mapped pinned host memory, a peer's page mapped through an IPC
 * handle) to `value` in stream order, behind everything enqueued on `stream`
 * so far. The word is then seen by kernels and CPUs of every process that has
 * the memory mapped. Stands in for cudaEventRecord on an inter-process event,
 * tensorpipe/channel/cuda_ipc/channel_impl.cc:238-252 (exporting a HIP event
 * to another process is refused where this library was built). */
int tphip_stream_signal(int dev, void* stream, void* word, uint64_t value);

/* tphip_batched_copy_signal behind a gate: a one-wavefront kernel enqueued
 * ahead of the copies waits, on the GPU, until the 64-bit word at `gate_word`
 * (readable by kernels of this device) has reached `gate_value`; the copy
 * kernels start when it has ended. The receiving half of tphip_stream_signal,
 * standing in for cudaStreamWaitEvent on an inter-process event,
 * tensorpipe/channel/cuda_ipc/channel_impl.cc:453-457. The wait is bounded:
 * if the word is not there after `max_wait_us` the gate raises the word at
 * `expired_word` (which the caller has zeroed; writable by kernels, readable
 * by the caller) to 1 and the copy kernels of the call do nothing, so the
 * stream always drains. Once `event` has completed the caller reads
 * *expired_word: non-zero means nothing was copied and the call must be
 * repeated. Up to 256 gated calls may be in flight per GPU. */
int tphip_batched_copy_gated(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                             void* event, const void* gate_word, uint64_t gate_value,
                             uint32_t max_wait_us, void* expired_word);

/* The resident copy agent: one workgroup that, once started, watches a ring
 * of commands in pinned host memory and performs small copies a few
 * microseconds after the host posted them -- no launch per copy. It starts
 * with the first submission, leaves by itself when nothing has come for
 * TPHIP_AGENT_IDLE_US (default 50) or after TPHIP_AGENT_LIFE_US (default
 * 1000) and is started again on demand; tphip_agent_destroy stops it and
 * waits for it. Copies are NOT ordered with any stream: the caller submits
 * only what is ready to be read and free to be written. The reference has no
 * counterpart (every one of its copies is a cudaMemcpyAsync). */
int tphip_agent_create(int dev, void** agent);
int tphip_agent_destroy(void* agent);
/* Posts the non-empty entries of table[0..n) (n <= 32) in order; *ticket
 * names the last one. After it has been copied, and made visible to every
 * process, `notify` (may be NULL; same kinds of address as for
 * tphip_stream_signal) is raised to `notify_value` (< 2^48). Returns
 * TPHIP_ERR_BUSY, posting nothing, when the ring cannot take the table now. */
int tphip_agent_submit(void* agent, const tphip_copy_desc* table, uint32_t n, void* notify,
                       uint64_t notify_value, uint64_t* ticket);
/* *done = 1 once the command named by `ticket` (and all before it) has been
 * served. Call it until then: it also restarts an agent that left before it
 * saw the command. */
int tphip_agent_done(void* agent, uint64_t ticket, int* done);

/* ---- GPU-driven staging ring ------------------------------------------------ */

/* One end of a staging ring that kernels walk by themselves: `num_slots` slots
 * of `slot_bytes` in pinned host memory, and two 64-bit counters in pinned
 * host memory, `produced` (chunks written into the ring) and `consumed`
 * (chunks read out of it), counted over the life of the ring, zero at the
 * start. Both ends -- normally two processes -- have slots and counters mapped
 * on their GPU (an IPC handle for the other side's memory). tphip_ring_push
 * enqueues ONE kernel that copies `bytes` bytes from `src` into the ring,
 * chunk by chunk (a chunk is one slot, the last may be shorter), waiting on
 * the GPU for `consumed` before it reuses a slot and raising `produced` behind
 * every chunk; tphip_ring_pull is the other half: it waits for `produced`,
 * copies slot -> `dst`, raises `consumed`. `first_seq` is the ring sequence
 * number of the call's first chunk (the total of all chunks moved before).
 * Replaces the per-chunk cudaMemcpyAsync + stream callback + control messages
 * of tensorpipe/channel/cuda_basic/channel_impl.cc:117-229 (send) and
 * :380-506 (recv).
 *
 * The kernels never wait for good: when nothing has moved for `yield_us`, or
 * the host has made *abort non-zero, the kernel leaves. Once `event` has
 * completed, *status (pinned host memory of this process) holds the ring
 * sequence number up to which this end is complete, with TPHIP_RING_YIELDED set
 * if the kernel left early; the caller then calls again for the rest
 * (src/dst and bytes advanced by the chunks done, first_seq = that number).
 * `scratch` is device memory of this end's own, tphip_ring_scratch_bytes()
 * long and zero before the first call; one call at a time per end. */
#define TPHIP_RING_YIELDED (1ull << 63)
typedef struct tphip_ring_end {
  void* slots;
  uint64_t slot_bytes;
  uint32_t num_slots;
  void* produced;
  void* consumed;
  void* scratch;
  void* status;
  const void* abort;
} tphip_ring_end;
size_t tphip_ring_scratch_bytes(uint32_t num_slots);
/* `blocks` workgroups of 256 threads (0 = the library's choice). */
int tphip_ring_push(int dev, const tphip_ring_end* ring, const void* src, uint64_t bytes,
                    uint64_t first_seq, uint32_t yield_us, uint32_t blocks, void* stream, void* event);
int tphip_ring_pull(int dev, const tphip_ring_end* ring, void* dst, uint64_t bytes,
                    uint64_t first_seq, uint32_t yield_us, uint32_t blocks, void* stream, void* event);

/* Single-copy convenience wrapper over the same kernel (n == 1, descriptor
 * travels in the kernel arguments). */
int tphip_copy(int dev, void* dst, const void* src, uint64_t bytes, void* stream);

/* Same as tphip_batched_copy with explicit launch shape, for tuning sweeps:
 * `unroll` in {1,2,4,8} 16-byte vectors in flight per lane, `blocks` workgroups
 * of 256 threads (0 = default: one per CU), `nontemporal` a mask (bit 0 =
 * nontemporal loads, bit 1 = nontemporal stores; negative = the default, which
 * goes by the bytes of the launch: 0 up to 64 MiB, up to 128 MiB 2 for a single entry and 0
 * for a table, 3 above). */
int tphip_batched_copy_tuned(int dev, const tphip_copy_desc* table, uint32_t n, void* stream,
                             int unroll, uint32_t blocks, int nontemporal);

/* Device-time measurement of the copy launches themselves. After
 * tphip_profile_start every tphip_batched_copy / tphip_copy launch on `dev` is
 * bracketed by two timing events on its own stream (up to `max_launches`, the
 * rest are counted but not timed); tphip_profile_stop waits for them and
 * reports how many launches were timed, their summed device time and the
 * payload bytes they moved. Profiling serialises nothing and is off by
 * default. The reference has no counterpart (it has no kernels). */
int tphip_profile_start(int dev, uint32_t max_launches);
int tphip_profile_stop(int dev, uint32_t* launches, double* total_ms, uint64_t* total_bytes);

/* Measurement only: a kernel that only reads (`write` == 0) or only writes
 * `bytes` bytes at `ptr` (device memory, 16-byte aligned) with the copy
 * kernels' access pattern and launch shape, eight vectors in flight per lane.
 * The two rates bound what a copy, which does both, can reach. The reference has
 * no counterpart. */
int tphip_bench_stream(int dev, int write, void* ptr, uint64_t bytes, void* stream);

/* Runtime copy engine path (hipMemcpyAsync), kept only as the A/B comparison
 * for the kernel-driven copies; the channels use it only when asked to
 * (TP_HIP_BASIC_ENGINE=sdma|mixed), never by default. */
int tphip_memcpy_async(int dev, void* dst, const void* src, uint64_t bytes, void* stream);

/* Fill `bytes` bytes at `ptr` with `value` using a kernel (safe to capture in
 * a HIP graph, unlike a memset node). */
int tphip_fill(int dev, void* ptr, int value, uint64_t bytes, void* stream);

/* Keeps `stream` busy for a long time while repeatedly rewriting `ptr[0..n)`,
 * leaving garbage behind; lets a test detect a missing event wait. HIP
 * counterpart of slowKernel, tensorpipe/test/channel/kernel.cu:11-22. */
int tphip_test_slow_kernel(int dev, void* ptr, uint64_t n, void* stream);

/* Test hook: the largest number of 16-byte vectors one table launch may
 * carry (its prefix sums are 32-bit); a table beyond it is cut into several
 * launches and an entry beyond it goes to the single-entry kernel. 0 restores
 * the built-in limit (just under 2^32 vectors = 64 GiB). Lets a test drive
 * the cut with small tables. The reference has no counterpart. */
int tphip_test_set_table_limit(uint64_t vectors);

#ifdef __cplusplus
}
#endif
#endif /* TPHIP_H_ */
