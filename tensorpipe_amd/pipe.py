"""Python face of the pipe/channel layer (C harness API in include/tensorpipe_c.h).

Mirrors the reference's usage pattern: a Context with registered transports and
channels, listen/connect, and Pipe.write / read_descriptor / read. Tensors are
described by (address, nbytes, device) with an explicit HIP stream for GPU
buffers, exactly what CpuBuffer / HipBuffer carry on the C++ side.
"""
import ctypes

import numpy as np

from . import _native

CPU, HIP, NO_TARGET = 0, 1, -1
MAX_DESC_ITEMS = 4096


class Tensor(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("length", ctypes.c_uint64),
        ("device_type", ctypes.c_int32),
        ("target_type", ctypes.c_int32),
        ("target_index", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("stream", ctypes.c_void_p),
    ]


class Payload(ctypes.Structure):
    _fields_ = [("ptr", ctypes.c_void_p), ("length", ctypes.c_uint64)]


class Descriptor(ctypes.Structure):
    _fields_ = [
        ("num_payloads", ctypes.c_uint32),
        ("num_tensors", ctypes.c_uint32),
        ("metadata", ctypes.c_char * 8192),
        ("payload_lengths", ctypes.c_uint64 * 64),
        ("tensor_lengths", ctypes.c_uint64 * MAX_DESC_ITEMS),
        ("tensor_source_type", ctypes.c_int32 * MAX_DESC_ITEMS),
        ("tensor_source_index", ctypes.c_int32 * MAX_DESC_ITEMS),
        ("tensor_target_type", ctypes.c_int32 * MAX_DESC_ITEMS),
        ("tensor_target_index", ctypes.c_int32 * MAX_DESC_ITEMS),
    ]


class PipeError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        _native.tphip()  # dependency, loaded first with RTLD_GLOBAL
        l = _native._load("libtensorpipe_amd.so")
        vp, i32, u32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint32
        P = ctypes.POINTER
        l.tpc_last_error.restype = ctypes.c_char_p
        l.tpc_context_create.restype = vp
        l.tpc_context_create.argtypes = [ctypes.c_char_p] * 3
        l.tpc_context_create_ex.restype = vp
        l.tpc_context_create_ex.argtypes = [ctypes.c_char_p] * 3 + [ctypes.c_int]
        l.tpc_context_close.argtypes = [vp]
        l.tpc_context_destroy.argtypes = [vp]
        l.tpc_context_has_channel.argtypes = [vp, ctypes.c_char_p]
        l.tpc_listen.restype = vp
        l.tpc_listen.argtypes = [vp, ctypes.c_char_p]
        l.tpc_listener_url.argtypes = [vp, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t]
        l.tpc_accept.restype = vp
        l.tpc_accept.argtypes = [vp, i32]
        l.tpc_listener_destroy.argtypes = [vp]
        l.tpc_connect.restype = vp
        l.tpc_connect.argtypes = [vp, ctypes.c_char_p]
        l.tpc_pipe_close.argtypes = [vp]
        l.tpc_pipe_destroy.argtypes = [vp]
        l.tpc_pipe_remote_name.argtypes = [vp, ctypes.c_char_p, ctypes.c_size_t]
        l.tpc_pipe_transport.argtypes = [vp, ctypes.c_char_p, ctypes.c_size_t]
        l.tpc_write_async.restype = vp
        l.tpc_write_async.argtypes = [vp, ctypes.c_char_p, P(Payload), u32, P(Tensor), u32]
        l.tpc_read_descriptor.argtypes = [vp, P(Descriptor), i32]
        l.tpc_read_async.restype = vp
        l.tpc_read_async.argtypes = [vp, P(vp), u32, P(Tensor), u32]
        l.tpc_op_wait.argtypes = [vp, i32]
        bench_args = [P(Payload), u32, P(vp), P(Tensor), P(Tensor), u32, u32, u32,
                      P(ctypes.c_double), P(ctypes.c_double)]
        l.tpc_bench_transfer.argtypes = [vp, vp] + bench_args
        l.tpc_bench_pingpong.argtypes = [vp, i32] + bench_args
        _lib = l
    return _lib


def _fail(what):
    raise PipeError(f"{what}: {lib().tpc_last_error().decode(errors='replace')}")


def _addr(x):
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    if isinstance(x, np.ndarray):
        return x.ctypes.data
    return int(x)


def make_tensor(buf, nbytes=None, device=None, stream=None, target=None):
    """Describe one tensor. `buf` is a torch tensor, a numpy array or an address.
    device: CPU or HIP (inferred for torch tensors / numpy arrays).
    target: None, or (device_type, index) the receiver must allocate on."""
    if device is None:
        device = HIP if (hasattr(buf, "is_cuda") and buf.is_cuda) else CPU
    if nbytes is None:
        nbytes = buf.numel() * buf.element_size() if hasattr(buf, "numel") else buf.nbytes
    if device == HIP and stream is None:
        import torch

        stream = torch.cuda.current_stream().cuda_stream
    if hasattr(stream, "cuda_stream"):
        stream = stream.cuda_stream
    t = Tensor()
    t.ptr = _addr(buf)
    t.length = int(nbytes)
    t.device_type = device
    if target is None:
        t.target_type, t.target_index = NO_TARGET, 0
    else:
        t.target_type, t.target_index = target
    t.stream = stream if device == HIP else None
    return t


def _tensor_array(tensors):
    arr = (Tensor * max(len(tensors), 1))()
    for i, t in enumerate(tensors):
        arr[i] = t
    return arr


def _payload_array(payloads):
    arr = (Payload * max(len(payloads), 1))()
    keep = []
    for i, p in enumerate(payloads):
        if isinstance(p, (bytes, bytearray)):
            b = (ctypes.c_char * max(len(p), 1)).from_buffer_copy(bytes(p) or b"\0")
            keep.append(b)
            arr[i].ptr = ctypes.addressof(b)
            arr[i].length = len(p)
        else:
            arr[i].ptr = _addr(p)
            arr[i].length = p.nbytes
            keep.append(p)
    return arr, keep


class Op:
    def __init__(self, handle, keep):
        if not handle:
            _fail("operation could not be started")
        self._h = handle
        self._keep = keep

    def wait(self, timeout_ms=30000):
        rc = lib().tpc_op_wait(self._h, timeout_ms)
        if rc != 0:
            _fail("operation failed" if rc == -1 else "operation timed out")
        self._keep = None


class Pipe:
    def __init__(self, handle):
        if not handle:
            _fail("pipe could not be created")
        self._h = handle

    def write(self, tensors=(), payloads=(), metadata=""):
        tarr = _tensor_array(list(tensors))
        parr, keep = _payload_array(list(payloads))
        h = lib().tpc_write_async(
            self._h, metadata.encode(), parr, len(payloads), tarr, len(tensors))
        return Op(h, (tarr, parr, keep, tensors))

    def read_descriptor(self, timeout_ms=30000):
        d = Descriptor()
        rc = lib().tpc_read_descriptor(self._h, ctypes.byref(d), timeout_ms)
        if rc != 0:
            _fail("readDescriptor")
        return d

    def read(self, tensors=(), payload_buffers=()):
        tarr = _tensor_array(list(tensors))
        pptrs = (ctypes.c_void_p * max(len(payload_buffers), 1))()
        for i, p in enumerate(payload_buffers):
            pptrs[i] = _addr(p)
        h = lib().tpc_read_async(self._h, pptrs, len(payload_buffers), tarr, len(tensors))
        return Op(h, (tarr, pptrs, payload_buffers, tensors))

    def remote_name(self):
        buf = ctypes.create_string_buffer(256)
        lib().tpc_pipe_remote_name(self._h, buf, 256)
        return buf.value.decode()

    def transport(self):
        """The transport the pipe runs on once the handshake is over ("" before)."""
        buf = ctypes.create_string_buffer(64)
        lib().tpc_pipe_transport(self._h, buf, 64)
        return buf.value.decode()

    def close(self):
        lib().tpc_pipe_close(self._h)

    def destroy(self):
        if self._h:
            lib().tpc_pipe_destroy(self._h)
            self._h = None


class Listener:
    def __init__(self, handle):
        if not handle:
            _fail("listen")
        self._h = handle

    def url(self, transport="shm"):
        buf = ctypes.create_string_buffer(512)
        if lib().tpc_listener_url(self._h, transport.encode(), buf, 512) != 0:
            _fail("listener url")
        return buf.value.decode()

    def accept(self, timeout_ms=30000):
        return Pipe(lib().tpc_accept(self._h, timeout_ms))

    def destroy(self):
        if self._h:
            lib().tpc_listener_destroy(self._h)
            self._h = None


class Context:
    """transports / channels: e.g. "shm:0" and "basic:0,hip_xth:10"."""

    def __init__(self, name="", transports="shm:0", channels="basic:0", stock_wire=None):
        """`transports` may name "uv" (TCP, framed like the reference's uv transport); `stock_wire`
        True puts the reference's own encodings on the wire, so that the peer may be an unmodified
        TensorPipe (None: as TP_STOCK_WIRE in the environment says)."""
        self._h = lib().tpc_context_create_ex(name.encode(), transports.encode(), channels.encode(),
                                              -1 if stock_wire is None else int(bool(stock_wire)))
        if not self._h:
            _fail("context")

    def has_channel(self, name):
        return bool(lib().tpc_context_has_channel(self._h, name.encode()))

    def listen(self, url="shm://"):
        """One URL, or several separated by commas: one listener per transport (a pipe opened on
        one of them moves to the best transport both ends have)."""
        return Listener(lib().tpc_listen(self._h, url.encode()))

    def connect(self, url):
        return Pipe(lib().tpc_connect(self._h, url.encode()))

    def close(self):
        lib().tpc_context_close(self._h)

    def destroy(self):
        if self._h:
            lib().tpc_context_destroy(self._h)
            self._h = None


def bench_transfer(sender, receiver, send_tensors, recv_tensors, payloads=(), recv_payloads=(),
                   warmup=5, iters=50):
    """Native timing loop (tpc_bench_transfer). Returns (per_iter_us ndarray, total_seconds)."""
    st, rt = _tensor_array(list(send_tensors)), _tensor_array(list(recv_tensors))
    parr, keep = _payload_array(list(payloads))
    pptrs = (ctypes.c_void_p * max(len(recv_payloads), 1))()
    for i, p in enumerate(recv_payloads):
        pptrs[i] = _addr(p)
    per = (ctypes.c_double * iters)()
    total = ctypes.c_double()
    rc = lib().tpc_bench_transfer(
        sender._h, receiver._h, parr, len(payloads), pptrs, st, rt, len(send_tensors),
        warmup, iters, per, ctypes.byref(total))
    if rc != 0:
        _fail("bench_transfer")
    return np.array(per[:]), total.value


def bench_pingpong(pipe, initiator, send_tensors, recv_tensors, payloads=(), recv_payloads=(),
                   warmup=5, iters=50):
    """initiator: False/0 echo side, True/1 initiator, 2 initiator whose wait for the receive
    streams runs on a thread of the chain's own (several chains side by side on one context)."""
    st, rt = _tensor_array(list(send_tensors)), _tensor_array(list(recv_tensors))
    parr, keep = _payload_array(list(payloads))
    pptrs = (ctypes.c_void_p * max(len(recv_payloads), 1))()
    for i, p in enumerate(recv_payloads):
        pptrs[i] = _addr(p)
    per = (ctypes.c_double * iters)()
    total = ctypes.c_double()
    rc = lib().tpc_bench_pingpong(
        pipe._h, int(initiator), parr, len(payloads), pptrs, st, rt, len(send_tensors),
        warmup, iters, per, ctypes.byref(total))
    if rc != 0:
        _fail("bench_pingpong")
    return np.array(per[:]), total.value
