"""The entry point that allocates nothing, mf_xcopy_device_table_static, against the entry point it
is a variant of, mf_xcopy_device_table: same destination bytes (bit-exact, whole destination pool
compared), on two calls in a row, the second with a smaller table, plus the limit and the oracle;
calls on two streams in turn; and the call captured into a HIP graph and replayed."""

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from tests import gpu_util

pytestmark = pytest.mark.gpu

MIB = 1 << 20
POOL = 64 * MIB


@pytest.fixture(scope="module")
def gpu(lib):
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    yield lib
    lib.hybm_uninit()


def _triples(base, src, dst, lens):
    t = np.empty((len(lens), 3), dtype=np.uint64)
    t[:, 0] = base + src
    t[:, 1] = base + dst
    t[:, 2] = lens
    return t.view(np.uint8).reshape(-1)


def test_static_scratch_entry_point_matches_the_allocating_one(gpu, oracle):
    init = np.empty(POOL, dtype=np.uint8)
    oracle.orc_fill_random(init.ctypes.data, POOL, 0x5C)
    pool = gpu_util.DeviceBuffer(gpu, POOL)
    table = gpu_util.DeviceBuffer(gpu, 24 * 32768)
    stream = gpu.mfrt_stream_create()
    try:
        # second call smaller than the first: what the first left in the scratch must not matter
        for count, seed, max_len in ((20000, 71, 1500), (300, 72, 60000), (1, 73, 5000)):
            src, dst, lens = workloads.ragged_batch(seed, POOL, count, max_len=max_len)
            table.upload(_triples(pool.ptr, src, dst, lens))
            results = []
            for entry in (gpu.mf_xcopy_device_table, gpu.mf_xcopy_device_table_static):
                pool.upload(init)
                assert entry(table.ptr, count, native.ROUTE_HBM, stream) == 0, native.last_error()
                assert gpu.mfrt_stream_sync(stream) == 0
                results.append(pool.download())
            assert np.array_equal(results[0], results[1]), f"{count} segments: the two entry points differ"
            expect = init.copy()
            gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
            assert np.array_equal(results[1], expect), f"{count} segments: differs from the oracle"
        # the limit is an error, not a silent truncation; an empty table is a no-op
        assert gpu.mf_xcopy_device_table_static(table.ptr, 32769, native.ROUTE_HBM, stream) == native.BM_INVALID_PARAM
        assert gpu.mf_xcopy_device_table_static(table.ptr, 0, native.ROUTE_HBM, stream) == 0
        assert gpu.mf_xcopy_device_table_static(None, 5, native.ROUTE_HBM, stream) == native.BM_INVALID_PARAM
        assert gpu.mfrt_stream_sync(stream) == 0
    finally:
        gpu.mfrt_stream_destroy(stream)
        table.free()
        pool.free()


def test_calls_on_two_streams_in_turn_are_kept_apart(gpu, oracle):
    """Every call uses the one scratch array of the GPU.  Calls that come on different streams, each reading what the one
    before wrote, are ordered by the library (an event behind every call, waited for by a call on another stream)."""
    init = np.empty(POOL, dtype=np.uint8)
    oracle.orc_fill_random(init.ctypes.data, POOL, 0x5D)
    pool = gpu_util.DeviceBuffer(gpu, POOL)
    tables = [gpu_util.DeviceBuffer(gpu, 24 * 4096) for _ in range(6)]
    streams = [gpu.mfrt_stream_create(), gpu.mfrt_stream_create()]
    try:
        pool.upload(init)
        expect = init.copy()
        region = POOL // 8
        for step, table in enumerate(tables):
            # step i moves 3000 ragged pieces from region i to region i + 1: a chain through the pool
            src, dst, lens = workloads.ragged_batch(80 + step, 2 * region, 3000, max_len=2500)
            src = src + step * region
            dst = dst - region + (step + 1) * region
            table.upload(_triples(pool.ptr, src, dst, lens))
            assert gpu.mf_xcopy_device_table_static(table.ptr, 3000, native.ROUTE_HBM, streams[step % 2]) == 0, native.last_error()
            snapshot = expect.copy()
            gpu_util.oracle_batch(oracle, snapshot, expect, src, dst, lens)
        assert gpu.mfrt_stream_sync(streams[0]) == 0 and gpu.mfrt_stream_sync(streams[1]) == 0
        assert np.array_equal(pool.download(), expect)
    finally:
        for s in streams:
            gpu.mfrt_stream_destroy(s)
        for t in tables:
            t.free()
        pool.free()


def test_static_entry_point_captured_in_a_graph_and_replayed(gpu, oracle):
    """What the entry point is for: a caller under HIP graph capture.  After one plain call (every kernel of the library has
    to have been launched once before anything is captured) the call is captured and the graph replayed three times, with
    fresh pool contents, eager copies and synchronisations between the replays; every replay against the oracle."""
    torch = pytest.importorskip("torch")
    assert torch.cuda.is_available()
    pool = gpu_util.DeviceBuffer(gpu, POOL)
    table = gpu_util.DeviceBuffer(gpu, 24 * 32768)
    stream = torch.cuda.Stream()
    raw = stream.cuda_stream
    try:
        for count, seed, kind in ((9000, 91, "ragged"), (700, 92, "pages")):
            if kind == "ragged":
                src, dst, lens = workloads.ragged_batch(seed, POOL, count, max_len=3000)
            else:   # equal pages: the planner finds the repeating chunk counts, the copy takes the form without a prefix
                rng = np.random.default_rng(seed)
                src = rng.permutation(count).astype(np.uint64) * np.uint64(32768)
                dst = np.uint64(POOL // 2) + rng.permutation(count).astype(np.uint64) * np.uint64(32768)
                lens = np.full(count, 20000, dtype=np.uint64)
            table.upload(_triples(pool.ptr, src, dst, lens))
            assert gpu.mf_xcopy_device_table_static(table.ptr, count, native.ROUTE_HBM, raw) == 0, native.last_error()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                ret = gpu.mf_xcopy_device_table_static(table.ptr, count, native.ROUTE_HBM, raw)
            assert ret == 0, native.last_error()
            for replay in range(3):
                init = np.empty(POOL, dtype=np.uint8)
                oracle.orc_fill_random(init.ctypes.data, POOL, seed * 10 + replay)
                pool.upload(init)
                graph.replay()
                torch.cuda.synchronize()
                got = pool.download()
                expect = init.copy()
                gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
                assert np.array_equal(got, expect), f"{kind}: replay {replay} differs from the oracle"
                # eager work of the same library between the replays
                assert gpu.mf_xcopy_device_table(table.ptr, count, native.ROUTE_HBM, None) == 0
                assert gpu.mfrt_device_sync() == 0
            del graph
    finally:
        table.free()
        pool.free()
