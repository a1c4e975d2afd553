"""ctypes bindings of the C-ABI libraries built in-tree.

Nothing here falls back to a CPU implementation: if a library is missing the
import of the symbol raises, so a GPU box can never silently run without the
HIP path.
"""
import ctypes
import os

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")


class NativeLibraryMissing(RuntimeError):
    pass


def lib_path(name):
    return os.path.join(_LIB_DIR, name)


def _load(name, mode=ctypes.DEFAULT_MODE):
    path = lib_path(name)
    if not os.path.exists(path):
        raise NativeLibraryMissing(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "at the repository root"
        )
    return ctypes.CDLL(path, mode=mode)


_hip_runtime_pinned = False


def _share_hip_runtime_with_torch():
    """One HIP runtime per process.

    PyTorch wheels bundle their own libamdhip64.so and link it by file name, while
    libtphip.so links the runtime by its soname (libamdhip64.so.7). If libtphip.so is
    loaded first, the system runtime comes in under the soname and a later `import torch`
    loads the bundled file as well: two runtimes, each blind to the other's allocations
    (pointer queries and hipIpcOpenMemHandle then fail with "invalid argument"). Loading
    the bundled runtime first, by path, makes both names resolve to that one object.
    Processes without torch simply get the system runtime.
    """
    global _hip_runtime_pinned
    if _hip_runtime_pinned:
        return
    _hip_runtime_pinned = True
    import importlib.util
    import sys

    if "torch" in sys.modules:
        return  # already loaded; libtphip.so binds to the same soname
    try:
        spec = importlib.util.find_spec("torch")
    except (ImportError, ValueError):
        spec = None
    if spec is None or not spec.origin:
        return
    bundled = os.path.join(os.path.dirname(spec.origin), "lib", "libamdhip64.so")
    if os.path.exists(bundled):
        ctypes.CDLL(bundled, mode=ctypes.RTLD_GLOBAL)


class CopyDesc(ctypes.Structure):
    """Mirror of tphip_copy_desc (include/tphip.h)."""

    _fields_ = [("src", ctypes.c_void_p), ("dst", ctypes.c_void_p), ("bytes", ctypes.c_uint64)]


class RingEnd(ctypes.Structure):
    """Mirror of tphip_ring_end (include/tphip.h)."""

    _fields_ = [("slots", ctypes.c_void_p), ("slot_bytes", ctypes.c_uint64), ("num_slots", ctypes.c_uint32),
                ("produced", ctypes.c_void_p), ("consumed", ctypes.c_void_p), ("scratch", ctypes.c_void_p),
                ("status", ctypes.c_void_p), ("abort", ctypes.c_void_p)]


_tphip = None
_datagen = None
_tpc = None


def tphip():
    global _tphip
    if _tphip is None:
        _share_hip_runtime_with_torch()
        lib = _load("libtphip.so", mode=ctypes.RTLD_GLOBAL)
        vp, i32, u32, u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64
        P = ctypes.POINTER
        lib.tphip_strerror.restype = ctypes.c_char_p
        lib.tphip_strerror.argtypes = [i32]
        lib.tphip_device_count.argtypes = [P(i32)]
        lib.tphip_device_uuid.argtypes = [i32, ctypes.c_char_p]
        lib.tphip_device_for_ptr.argtypes = [vp, P(i32), P(i32)]
        lib.tphip_mem_base.argtypes = [vp, P(vp), P(ctypes.c_size_t)]
        lib.tphip_malloc.argtypes = [i32, ctypes.c_size_t, P(vp)]
        lib.tphip_free.argtypes = [i32, vp]
        lib.tphip_host_alloc.argtypes = [i32, ctypes.c_size_t, P(vp), P(vp)]
        lib.tphip_host_free.argtypes = [vp]
        lib.tphip_stream_create.argtypes = [i32, P(vp)]
        lib.tphip_stream_destroy.argtypes = [i32, vp]
        lib.tphip_stream_sync.argtypes = [i32, vp]
        lib.tphip_stream_query.argtypes = [i32, vp, P(i32)]
        lib.tphip_event_create.argtypes = [i32, i32, P(vp)]
        lib.tphip_event_create_timed.argtypes = [i32, P(vp)]
        lib.tphip_event_destroy.argtypes = [i32, vp]
        lib.tphip_event_record.argtypes = [i32, vp, vp]
        lib.tphip_stream_wait_event.argtypes = [i32, vp, vp]
        lib.tphip_event_query.argtypes = [i32, vp, P(i32)]
        lib.tphip_event_sync.argtypes = [i32, vp]
        lib.tphip_event_elapsed_ms.argtypes = [vp, vp, P(ctypes.c_float)]
        lib.tphip_ipc_mem_export.argtypes = [i32, vp, ctypes.c_char_p]
        lib.tphip_ipc_mem_open.argtypes = [i32, ctypes.c_char_p, P(vp)]
        lib.tphip_ipc_mem_close.argtypes = [i32, vp]
        lib.tphip_ipc_event_export.argtypes = [i32, vp, ctypes.c_char_p]
        lib.tphip_ipc_event_open.argtypes = [i32, ctypes.c_char_p, P(vp)]
        lib.tphip_batched_copy.argtypes = [i32, P(CopyDesc), u32, vp]
        lib.tphip_batched_copy_signal.argtypes = [i32, P(CopyDesc), u32, vp, vp, i32, u32, i32]
        lib.tphip_batched_copy_noalloc.argtypes = [i32, P(CopyDesc), u32, vp]
        lib.tphip_copy.argtypes = [i32, vp, vp, u64, vp]
        lib.tphip_stream_signal.argtypes = [i32, vp, vp, u64]
        lib.tphip_batched_copy_gated.argtypes = [i32, P(CopyDesc), u32, vp, vp, vp, u64, u32, vp]
        lib.tphip_agent_create.argtypes = [i32, P(vp)]
        lib.tphip_agent_destroy.argtypes = [vp]
        lib.tphip_agent_submit.argtypes = [vp, P(CopyDesc), u32, vp, u64, P(u64)]
        lib.tphip_agent_done.argtypes = [vp, u64, P(i32)]
        lib.tphip_batched_copy_tuned.argtypes = [i32, P(CopyDesc), u32, vp, i32, u32, i32]
        lib.tphip_profile_start.argtypes = [i32, u32]
        lib.tphip_profile_stop.argtypes = [i32, P(u32), P(ctypes.c_double), P(u64)]
        lib.tphip_mem_buffer_id.argtypes = [vp, P(u64)]
        lib.tphip_memcpy_async.argtypes = [i32, vp, vp, u64, vp]
        lib.tphip_fill.argtypes = [i32, vp, i32, u64, vp]
        lib.tphip_test_slow_kernel.argtypes = [i32, vp, u64, vp]
        lib.tphip_test_set_table_limit.argtypes = [u64]
        lib.tphip_bench_stream.argtypes = [i32, i32, vp, u64, vp]
        lib.tphip_ring_scratch_bytes.restype = ctypes.c_size_t
        lib.tphip_ring_scratch_bytes.argtypes = [u32]
        lib.tphip_ring_push.argtypes = [i32, P(RingEnd), vp, u64, u64, u32, u32, vp, vp]
        lib.tphip_ring_pull.argtypes = [i32, P(RingEnd), vp, u64, u64, u32, u32, vp, vp]
        _tphip = lib
    return _tphip


def datagen():
    global _datagen
    if _datagen is None:
        lib = _load("libtpdatagen.so")
        vp, u32, u64 = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64
        lib.tpdg_u64.restype = u64
        lib.tpdg_u64.argtypes = [u64, u64]
        lib.tpdg_fill_u8.argtypes = [u64, vp, u64]
        for name in ("tpdg_fill_normal_f32", "tpdg_fill_normal_bf16", "tpdg_fill_normal_f16"):
            getattr(lib, name).argtypes = [u64, ctypes.c_double, vp, u64]
        lib.tpdg_loguniform_sizes.argtypes = [u64, u64, u64, vp, u32]
        lib.tpdg_bench_pattern.argtypes = [vp, u64]
        lib.tpdg_fnv1a64.restype = u64
        lib.tpdg_fnv1a64.argtypes = [vp, u64]
        _datagen = lib
    return _datagen


class HipError(RuntimeError):
    def __init__(self, code, what):
        super().__init__(f"{what} failed: [{code}] {tphip().tphip_strerror(code).decode()}")
        self.code = code


def check(code, what="tphip call"):
    if code != 0:
        raise HipError(code, what)
