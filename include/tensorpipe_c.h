/*
 * tensorpipe_c.h -- C harness API over the C++ pipe/channel layer in
 * libtensorpipe_amd.so. The product API is the C++ one (tensorpipe::Context /
 * Listener / Pipe and the channel plugin surface); this header exists so that
 * tests, the smoke check and the bench can drive that API from Python (ctypes)
 * or C with plain pointers and sizes. Calls block until the corresponding C++
 * callback has fired (or the timeout expires), except where named _async.
 *
 * Return values: 0 = success, TPC_ERR_TIMEOUT, or TPC_ERR_FAILED; after a
 * failure tpc_last_error() returns the tensorpipe::Error::what() string (or
 * exception text) for the calling thread.
 *
 * Reference interfaces mirrored: tensorpipe/core/context.h:58-94 (register*,
 * listen, connect), tensorpipe/core/listener.h:56-83 (accept, url),
 * tensorpipe/core/pipe.h:66-84 (readDescriptor, read, write),
 * tensorpipe/core/message.h:27-102 (Message/Descriptor/Allocation fields).
 */
#ifndef TENSORPIPE_C_H_
#define TENSORPIPE_C_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TPC_ERR_FAILED (-1)
#define TPC_ERR_TIMEOUT (-2)

#define TPC_DEVICE_CPU 0
#define TPC_DEVICE_HIP 1
#define TPC_NO_TARGET (-1)

typedef struct tpc_context tpc_context;
typedef struct tpc_listener tpc_listener;
typedef struct tpc_pipe tpc_pipe;
typedef struct tpc_op tpc_op;

/* One tensor of a message (sender) or of an allocation (receiver).
 * device_type selects CpuBuffer{ptr} or HipBuffer{ptr, stream}; target_type is
 * TPC_NO_TARGET or the device type the receiver must allocate on. */
typedef struct tpc_tensor {
  void* ptr;
  uint64_t length;
  int32_t device_type;
  int32_t target_type;
  int32_t target_index;
  int32_t reserved;
  void* stream;
} tpc_tensor;

typedef struct tpc_payload {
  void* ptr;
  uint64_t length;
} tpc_payload;

#define TPC_MAX_DESC_ITEMS 4096

/* What readDescriptor delivers: counts, lengths and devices. */
typedef struct tpc_descriptor {
  uint32_t num_payloads;
  uint32_t num_tensors;
  char metadata[8192];
  uint64_t payload_lengths[64];
  uint64_t tensor_lengths[TPC_MAX_DESC_ITEMS];
  int32_t tensor_source_type[TPC_MAX_DESC_ITEMS];
  int32_t tensor_source_index[TPC_MAX_DESC_ITEMS];
  int32_t tensor_target_type[TPC_MAX_DESC_ITEMS];
  int32_t tensor_target_index[TPC_MAX_DESC_ITEMS];
} tpc_descriptor;

const char* tpc_last_error(void);

/* Context: `transports` and `channels` are comma-separated lists of
 * "name:priority" with names from {shm, uv} and {basic, xth, hip_xth, hip_ipc,
 * hip_basic}; hip_basic wraps a fresh basic context. */
tpc_context* tpc_context_create(const char* name, const char* transports, const char* channels);
/* The same with two more things to say: "uv" among the transports is this
 * library's TCP transport under the name a stock TensorPipe gives its own, and
 * stock_wire chooses the encodings on the wire (1: the reference's own, so
 * that the peer may be an unmodified TensorPipe; 0: this library's; -1: as
 * TP_STOCK_WIRE in the environment says). */
tpc_context* tpc_context_create_ex(const char* name, const char* transports, const char* channels, int stock_wire);
void tpc_context_close(tpc_context* ctx);
void tpc_context_destroy(tpc_context* ctx); /* join + free */
/* 1 if the named channel was viable and got registered. */
int tpc_context_has_channel(tpc_context* ctx, const char* name);

/* url: one URL, or several separated by commas (one listener per transport). */
tpc_listener* tpc_listen(tpc_context* ctx, const char* url);
int tpc_listener_url(tpc_listener* l, const char* transport, char* out, size_t out_len);
tpc_pipe* tpc_accept(tpc_listener* l, int timeout_ms);
void tpc_listener_destroy(tpc_listener* l);

tpc_pipe* tpc_connect(tpc_context* ctx, const char* url);
void tpc_pipe_close(tpc_pipe* p);
void tpc_pipe_destroy(tpc_pipe* p);
int tpc_pipe_remote_name(tpc_pipe* p, char* out, size_t out_len);
/* The transport the pipe's own connections run on after the handshake ("" before): the server
 * moves a pipe to the best transport both ends have (tensorpipe/core/pipe_impl.cc:987-1042,
 * 1108-1125). Not from a callback of the pipe. */
int tpc_pipe_transport(tpc_pipe* p, char* out, size_t out_len);

/* Pipe::write; returns an operation to wait on. Payload and tensor memory must
 * stay valid until the operation completed. */
tpc_op* tpc_write_async(tpc_pipe* p, const char* metadata, const tpc_payload* payloads,
                        uint32_t num_payloads, const tpc_tensor* tensors, uint32_t num_tensors);
/* Pipe::readDescriptor, blocking. */
int tpc_read_descriptor(tpc_pipe* p, tpc_descriptor* out, int timeout_ms);
/* Pipe::read for the descriptor delivered last; returns an operation. */
tpc_op* tpc_read_async(tpc_pipe* p, void* const* payload_ptrs, uint32_t num_payloads,
                       const tpc_tensor* tensors, uint32_t num_tensors);
/* Waits for the operation's callback, frees the operation, returns its status. */
int tpc_op_wait(tpc_op* op, int timeout_ms);

/* Benchmark loops run natively so that no interpreter time is on the clock.
 *
 * tpc_bench_transfer: `iters` times (after `warmup` untimed ones) send the
 * tensors from `sender` and receive them into `recv_tensors` on `receiver`
 * (both pipes in this process): write, readDescriptor, read, wait for both
 * callbacks, then synchronise every distinct receive stream. per_iter_us (may
 * be NULL) gets each iteration's wall time. Returns 0 or an error code. */
int tpc_bench_transfer(tpc_pipe* sender, tpc_pipe* receiver, const tpc_payload* payloads,
                       uint32_t num_payloads, void* const* recv_payload_ptrs,
                       const tpc_tensor* send_tensors, const tpc_tensor* recv_tensors,
                       uint32_t num_tensors, uint32_t warmup, uint32_t iters, double* per_iter_us,
                       double* total_seconds);

/* Ping-pong over one pipe, one endpoint per process (or thread):
 * the initiator writes the message and waits to read it back; the echo side
 * reads and writes back. Both sides pass their own buffers. The initiator's
 * per_iter_us receives round-trip times including the final stream
 * synchronisation (tensorpipe/benchmark/benchmark_pipe.cc:463-468,571-577).
 * initiator: 0 = echo side, 1 = initiator, 2 = initiator that waits for its
 * receive streams on a thread of the chain's own instead of the context's
 * (for several chains side by side on one context: a wait on the context's
 * thread would hold up every other chain's messages for a kernel's length). */
int tpc_bench_pingpong(tpc_pipe* p, int initiator, const tpc_payload* payloads,
                       uint32_t num_payloads, void* const* recv_payload_ptrs,
                       const tpc_tensor* send_tensors, const tpc_tensor* recv_tensors,
                       uint32_t num_tensors, uint32_t warmup, uint32_t iters, double* per_iter_us,
                       double* total_seconds);

#ifdef __cplusplus
}
#endif
#endif /* TENSORPIPE_C_H_ */
