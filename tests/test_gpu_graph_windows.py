"""A copy large enough for read and write windows, captured into a HIP graph and replayed.  The waves of a windowed
launch agree on the start of their schedule through a device word that carries the launch's sequence number; a replay
carries the number it was captured with and must still find a fresh start (or run unpaced), never the start of the
replay before it.  Every replay is compared with the slices cut on the CPU."""

import numpy as np
import pytest

from memfabric_hybrid_amd import native
from tests import gpu_util

pytestmark = pytest.mark.gpu

MIB = 1 << 20


@pytest.fixture(scope="module")
def gpu(lib):
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    yield lib
    lib.hybm_uninit()


@pytest.mark.parametrize("layout", ["on-cache-lines", "between-cache-lines"])
def test_windowed_copy_captured_in_a_graph_and_replayed(gpu, oracle, layout):
    torch = pytest.importorskip("torch")
    assert torch.cuda.is_available()
    half = 256 * MIB
    pool = gpu_util.DeviceBuffer(gpu, 2 * half)
    stream = torch.cuda.Stream()
    raw = stream.cuda_stream
    shift = 0 if layout == "on-cache-lines" else 48
    # three segments, 200 MiB in all (12 800 chunks of 16 KiB: four periods on 3200 waves), destinations in another order
    lens = np.array([90 * MIB, 10 * MIB + 4096, 100 * MIB - 4096], dtype=np.uint64)
    src = np.array([shift, 100 * MIB + shift, 120 * MIB + shift], dtype=np.uint64)
    dst = np.array([half + 110 * MIB + shift, half + shift, half + 10 * MIB + 8192 + shift], dtype=np.uint64)
    args = (native.u64_array(pool.ptr + src), native.u64_array(pool.ptr + dst), native.u64_array(lens), 3, native.ROUTE_HBM, raw)
    try:
        # once plainly: every kernel of the library has been launched before anything is captured
        assert gpu.mf_xcopy_batch(*args) == 0, native.last_error()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            ret = gpu.mf_xcopy_batch(*args)
        assert ret == 0, native.last_error()
        block = np.empty(64 * MIB, dtype=np.uint8)
        for replay in range(3):
            oracle.orc_fill_random(block.ctypes.data, len(block), 0x600 + replay)
            for i in range(0, half, len(block)):
                pool.upload(block ^ np.uint8(i // len(block) + 1), offset=i)
            assert gpu.mfrt_memset(pool.ptr + half, 0x5A, half) == 0
            assert gpu.mfrt_device_sync() == 0
            graph.replay()
            torch.cuda.synchronize()
            got = pool.download(offset=half)
            expect = np.full(half, 0x5A, dtype=np.uint8)
            for s, d, n in zip(src.tolist(), dst.tolist(), lens.tolist()):
                for i in range(0, n, len(block)):       # the source, rebuilt block by block
                    m = min(len(block), n - i)
                    at = s + i
                    b0 = at // len(block)
                    off = at - b0 * len(block)
                    first = min(m, len(block) - off)
                    expect[d - half + i:d - half + i + first] = block[off:off + first] ^ np.uint8(b0 + 1)
                    if first < m:
                        expect[d - half + i + first:d - half + i + m] = block[:m - first] ^ np.uint8(b0 + 2)
            assert np.array_equal(got, expect), f"replay {replay} differs"
            # eager work of the same kind between the replays: its sequence numbers move on, the graph's do not
            assert gpu.mf_xcopy_batch(args[0], args[1], args[2], 3, native.ROUTE_HBM, None) == 0
            assert gpu.mfrt_device_sync() == 0
        del graph
    finally:
        pool.free()
