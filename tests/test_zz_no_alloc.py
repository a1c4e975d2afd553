"""tphip_batched_copy_noalloc (the entry point that allocates nothing, plan in a device array of
the library image) against tphip_batched_copy on the same tables, through the C ABI: byte-identical
destinations, and against the CPU oracle. Two calls in a row share the array; the second one is
smaller than the first."""
import ctypes

import numpy as np
import pytest

from tensorpipe_amd import _native, datagen, hip

pytestmark = pytest.mark.gpu

FILL = 0xEE


def _layout(sizes, seed):
    rng = np.random.default_rng(seed)
    layout, so, do = [], 0, 0
    for n in sizes:
        so = (so + 15) // 16 * 16 + int(rng.integers(0, 16))
        do = (do + 15) // 16 * 16 + int(rng.integers(0, 16))
        layout.append((so, do, int(n)))
        so += int(n) + 24
        do += int(n) + 24
    return layout, so + 64, do + 64


def _both_ways(oracle, sizes, seed):
    """Runs one table through both entry points; returns nothing, asserts equality."""
    import torch

    lib = _native.tphip()
    layout, src_size, dst_size = _layout(sizes, seed)
    host_src = datagen.uniform_u8(seed, src_size)
    src = torch.from_numpy(host_src).cuda()
    dst_new = torch.full((dst_size,), FILL, dtype=torch.uint8, device="cuda")
    dst_old = torch.full((dst_size,), FILL, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()

    table, n = hip.make_table([(src.data_ptr() + s, dst_new.data_ptr() + d, b) for s, d, b in layout])
    _native.check(lib.tphip_batched_copy_noalloc(0, table, n, stream), "tphip_batched_copy_noalloc")
    table2, n2 = hip.make_table([(src.data_ptr() + s, dst_old.data_ptr() + d, b) for s, d, b in layout])
    _native.check(lib.tphip_batched_copy(0, table2, n2, stream), "tphip_batched_copy")
    torch.cuda.synchronize()

    got_new = dst_new.cpu().numpy()
    got_old = dst_old.cpu().numpy()
    bad = np.nonzero(got_new != got_old)[0]
    assert bad.size == 0, f"{bad.size} bytes differ from tphip_batched_copy, first at {bad[0]}"
    ref = np.full(dst_size, FILL, dtype=np.uint8)
    oracle.xth_message([(host_src[s:], ref[d:], b) for s, d, b in layout])
    bad = np.nonzero(got_new != ref)[0]
    assert bad.size == 0, f"{bad.size} bytes differ from the oracle, first at {bad[0]}"
    assert (src.cpu().numpy() == host_src).all(), "source was modified"


def test_two_calls_in_a_row_the_second_smaller(oracle):
    big = [int(s) for s in datagen.loguniform_sizes(71, 1, 1 << 20, 700)] + [0, 1, 15, 16, 17]
    _both_ways(oracle, big, seed=7001)
    small = [int(s) for s in datagen.loguniform_sizes(72, 1, 1 << 16, 130)]
    _both_ways(oracle, small, seed=7002)
    # and down to the shapes that need no table at all in the other entry point
    _both_ways(oracle, [4099, 0, 77], seed=7003)
    _both_ways(oracle, [1 << 22], seed=7004)


def test_limits_and_empty_tables():
    import torch

    lib = _native.tphip()
    stream = torch.cuda.current_stream().cuda_stream
    a = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    b = torch.ones(4096, dtype=torch.uint8, device="cuda")
    table, n = hip.make_table([(b.data_ptr(), a.data_ptr(), 1)] * 1025)
    assert lib.tphip_batched_copy_noalloc(0, table, n, stream) == -2  # TPHIP_ERR_TOO_LARGE
    torch.cuda.synchronize()
    assert int(a.sum().item()) == 0, "a rejected call must enqueue nothing"
    assert lib.tphip_batched_copy_noalloc(0, table, 0, stream) == 0
    empty, n = hip.make_table([(b.data_ptr(), a.data_ptr(), 0)] * 5)
    assert lib.tphip_batched_copy_noalloc(0, empty, n, stream) == 0
    bad, n = hip.make_table([(0, a.data_ptr(), 16)])
    assert lib.tphip_batched_copy_noalloc(0, bad, n, stream) == -1  # TPHIP_ERR_INVALID_ARG
    torch.cuda.synchronize()
    assert int(a.sum().item()) == 0


def test_full_size_table(oracle):
    sizes = [int(s) for s in datagen.loguniform_sizes(73, 16, 1 << 14, 1024)]
    _both_ways(oracle, sizes, seed=7005)


def test_captured_in_a_graph_and_replayed(oracle):
    """The callers this entry point is for include code under stream capture: a captured call
    (plan pieces and table kernel, nothing else) copies on every replay what the sources hold
    then, with eager calls that overwrite the shared plan array in between."""
    import torch

    lib = _native.tphip()
    sizes = [int(s) for s in datagen.loguniform_sizes(74, 1, 1 << 18, 300)] + [0, 1, 15, 16, 17, 1 << 21]
    layout, src_size, dst_size = _layout(sizes, 7006)
    src = torch.zeros(src_size, dtype=torch.uint8, device="cuda")
    dst = torch.zeros(dst_size, dtype=torch.uint8, device="cuda")
    table, n = hip.make_table([(src.data_ptr() + s, dst.data_ptr() + d, b) for s, d, b in layout])
    # the device's array is looked up on the first call: that one stays outside the capture
    _native.check(lib.tphip_batched_copy_noalloc(0, table, n, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = torch.cuda.current_stream().cuda_stream
        _native.check(lib.tphip_batched_copy_noalloc(0, table, n, stream), "tphip_batched_copy_noalloc (capturing)")

    for replay in range(3):
        host_src = datagen.uniform_u8(7100 + replay, src_size)
        src.copy_(torch.from_numpy(host_src))
        dst.fill_(FILL)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref = np.full(dst_size, FILL, dtype=np.uint8)
        oracle.xth_message([(host_src[s:], ref[d:], b) for s, d, b in layout])
        bad = np.nonzero(dst.cpu().numpy() != ref)[0]
        assert bad.size == 0, f"replay {replay}: {bad.size} bytes differ from the oracle, first at {bad[0]}"
        # an eager call with another table leaves its own plan in the array before the next replay
        _both_ways(oracle, [333 + replay, 70000, 5], seed=7200 + replay)
