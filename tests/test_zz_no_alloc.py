"""The entry point that allocates nothing, mf_xcopy_device_table_static, against the entry point it
is a variant of, mf_xcopy_device_table: same destination bytes (bit-exact, whole destination pool
compared), on two calls in a row, the second with a smaller table, plus the limit and the oracle."""

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
