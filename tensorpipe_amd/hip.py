"""Python face of the tphip C ABI: the batched multi-tensor copy and the few
runtime calls tests and the bench need. Device memory and streams come from
PyTorch; every byte is moved by libtphip."""
import ctypes

from . import _native
from ._native import CopyDesc, check


def _ptr(x):
    return x.data_ptr() if hasattr(x, "data_ptr") else int(x)


def _nbytes(x):
    return x.numel() * x.element_size()


def _stream_handle(stream):
    if stream is None:
        import torch

        return torch.cuda.current_stream().cuda_stream
    return stream.cuda_stream if hasattr(stream, "cuda_stream") else int(stream)


def make_table(entries):
    """entries: iterable of (src, dst, nbytes) with torch tensors or raw addresses."""
    entries = list(entries)
    table = (CopyDesc * max(len(entries), 1))()
    for i, (src, dst, nbytes) in enumerate(entries):
        table[i].src = _ptr(src)
        table[i].dst = _ptr(dst)
        table[i].bytes = int(nbytes)
    return table, len(entries)


def batched_copy(entries, stream=None, device=0):
    """One launch for all (src, dst, nbytes) entries on `stream` (default: torch's current)."""
    table, n = make_table(entries)
    check(
        _native.tphip().tphip_batched_copy(device, table, n, _stream_handle(stream)),
        "tphip_batched_copy",
    )


def batched_copy_table(table, n, stream=None, device=0, unroll=None, blocks=0, nontemporal=1):
    lib = _native.tphip()
    if unroll is None:
        check(lib.tphip_batched_copy(device, table, n, _stream_handle(stream)), "tphip_batched_copy")
    else:
        check(
            lib.tphip_batched_copy_tuned(
                device, table, n, _stream_handle(stream), unroll, blocks, nontemporal
            ),
            "tphip_batched_copy_tuned",
        )


def copy(dst, src, nbytes=None, stream=None, device=0):
    if nbytes is None:
        nbytes = _nbytes(src)
    check(
        _native.tphip().tphip_copy(device, _ptr(dst), _ptr(src), nbytes, _stream_handle(stream)),
        "tphip_copy",
    )


def memcpy_async(dst, src, nbytes, stream=None, device=0):
    check(
        _native.tphip().tphip_memcpy_async(
            device, _ptr(dst), _ptr(src), nbytes, _stream_handle(stream)
        ),
        "tphip_memcpy_async",
    )


def device_count():
    n = ctypes.c_int(0)
    check(_native.tphip().tphip_device_count(ctypes.byref(n)), "tphip_device_count")
    return n.value


class TimedEvent:
    """Timing event recorded on an explicit stream handle (torch.cuda.Event only
    sees torch's current stream)."""

    def __init__(self, device=0):
        self.device = device
        h = ctypes.c_void_p()
        check(_native.tphip().tphip_event_create_timed(device, ctypes.byref(h)), "event_create")
        self.handle = h

    def record(self, stream=None):
        check(
            _native.tphip().tphip_event_record(self.device, self.handle, _stream_handle(stream)),
            "event_record",
        )

    def synchronize(self):
        check(_native.tphip().tphip_event_sync(self.device, self.handle), "event_sync")

    def elapsed_ms(self, later):
        ms = ctypes.c_float()
        check(
            _native.tphip().tphip_event_elapsed_ms(self.handle, later.handle, ctypes.byref(ms)),
            "event_elapsed",
        )
        return ms.value

    def __del__(self):
        try:
            _native.tphip().tphip_event_destroy(self.device, self.handle)
        except Exception:
            pass
