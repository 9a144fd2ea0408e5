"""GPU tests of the drop-in surfaces: smem_bm_* / hybm_* calls and the two-symbol copy plugin,
each compared with the CPU oracle."""

import ctypes
import os

import numpy as np
import pytest

from memfabric_hybrid_amd import bm, native, workloads
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

MIB = 1 << 20
POOL = 128 * MIB


@pytest.fixture(scope="module")
def pool(lib):
    assert bm.initialize("tcp://127.0.0.1:5432", 1, 0) == 0, native.last_error()
    handle = bm.create(3, POOL, POOL, bm.BmDataOpType.SDMA)
    assert handle.join() == 0
    yield handle
    handle.leave()
    handle.destroy()
    bm.uninitialize()


def _rand(oracle, n, seed):
    a = np.empty(n, dtype=np.uint8)
    oracle.orc_fill_random(np_ptr(a), n, seed)
    return a


def test_pool_layout(pool, lib):
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    assert dev and host
    assert pool.local_mem_size(bm.BmMemType.DEVICE) == POOL and pool.local_mem_size(bm.BmMemType.HOST) == POOL
    assert bm.bm_rank_id() == 0
    assert pool.get_rank_id_by_gva(dev) == 0 and pool.get_rank_id_by_gva(host + POOL - 1) == 0
    assert pool.get_rank_id_by_gva(host + POOL + 4096) == 0xFFFFFFFF
    assert lib.smem_bm_ptr_by_mem_type(pool.handle, native.SMEM_MEM_TYPE_DEVICE, 1) is None
    assert lib.mfrt_pointer_kind(dev) == native.PTR_DEVICE
    assert lib.mfrt_pointer_kind(host) == native.PTR_PINNED_HOST
    # the registry knows both pools: AUTO can classify
    assert lib.mf_va_infer_direction(host, dev) == native.HYBM_DIR["GH2GD"]
    assert lib.mf_va_infer_direction(dev + 5, dev + 99) == native.HYBM_DIR["GD2GD"]


def test_batch_copy_chain_h2g_g2g_g2h(pool, lib, oracle):
    """Host pool -> HBM pool -> elsewhere in HBM pool -> host pool, 122-segment batches, via
    smem_bm_copy_batch; mirrored step by step on CPU arrays with the oracle."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    hview = gpu_util.host_view(host, POOL)
    hview[:] = _rand(oracle, POOL, 0xD1)
    assert lib.mfrt_memset(dev, 0x33, POOL) == 0
    model_host = hview.copy()
    model_dev = np.full(POOL, 0x33, dtype=np.uint8)

    s1, d1, l1 = workloads.kv_batch(1, POOL, same_pool=False)
    assert pool.copy_data_batch((host + s1).tolist(), (dev + d1).tolist(), l1.tolist(), 122, bm.BmCopyType.G2G) == 0, \
        native.last_error()
    gpu_util.oracle_batch(oracle, model_host, model_dev, s1, d1, l1)

    s2, d2, l2 = workloads.kv_batch(2, POOL)
    snapshot = model_dev.copy()
    assert pool.copy_data_batch((dev + s2).tolist(), (dev + d2).tolist(), l2.tolist(), 122, bm.BmCopyType.AUTO) == 0
    gpu_util.oracle_batch(oracle, snapshot, model_dev, s2, d2, l2)

    s3, d3, l3 = workloads.kv_batch(3, POOL, same_pool=False)
    assert pool.copy_data_batch((dev + s3).tolist(), (host + d3).tolist(), l3.tolist(), 122, bm.BmCopyType.G2G,
                                native.COPY_EXTEND_FLAG) == 0
    gpu_util.oracle_batch(oracle, model_dev, model_host, s3, d3, l3)

    got_dev = np.empty(POOL, dtype=np.uint8)
    assert lib.mfrt_memcpy(np_ptr(got_dev), dev, POOL) == 0
    assert np.array_equal(got_dev, model_dev)
    assert np.array_equal(hview, model_host)


def test_single_copy_all_executable_directions(pool, lib, oracle):
    """smem_bm_copy with every copy type, local sides in pageable numpy memory, pinned memory
    and a private device buffer."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    hview = gpu_util.host_view(host, POOL)
    n = 3 * MIB + 17
    payload = _rand(oracle, n, 0xD2)
    local_dev = gpu_util.DeviceBuffer(lib, n + 64)
    pinned = gpu_util.PinnedBuffer(lib, n + 64)
    try:
        # H2G from pageable memory into the HBM pool, G2H back into pageable memory
        assert pool.copy_data(np_ptr(payload), dev + 4099, n, bm.BmCopyType.H2G) == 0, native.last_error()
        back = np.zeros(n, dtype=np.uint8)
        assert pool.copy_data(dev + 4099, np_ptr(back), n, bm.BmCopyType.G2H) == 0
        assert np.array_equal(back, payload)
        # H2G / G2H with pinned local memory (no staging)
        pinned.array[:n] = payload[::-1]
        assert pool.copy_data(pinned.ptr, dev + 8 * MIB + 1, n, bm.BmCopyType.H2G) == 0
        pinned.array[:] = 0
        assert pool.copy_data(dev + 8 * MIB + 1, pinned.ptr + 3, n, bm.BmCopyType.G2H) == 0
        assert np.array_equal(pinned.array[3:3 + n], payload[::-1])
        # L2G / G2L with a private device buffer
        local_dev.upload(payload)
        assert pool.copy_data(local_dev.ptr, dev + 16 * MIB + 7, n, bm.BmCopyType.L2G) == 0
        local_dev.fill(0)
        assert pool.copy_data(dev + 16 * MIB + 7, local_dev.ptr + 5, n, bm.BmCopyType.G2L) == 0
        assert np.array_equal(local_dev.download(5, n), payload)
        # H2GH / GH2H: pageable <-> host pool
        assert pool.copy_data(np_ptr(payload), host + 24 * MIB + 9, n, bm.BmCopyType.H2GH) == 0
        assert np.array_equal(hview[24 * MIB + 9:24 * MIB + 9 + n], payload)
        back[:] = 0
        assert pool.copy_data(host + 24 * MIB + 9, np_ptr(back), n, bm.BmCopyType.GH2H) == 0
        assert np.array_equal(back, payload)
        # G2G: device pool -> host pool -> device pool
        assert pool.copy_data(dev + 16 * MIB + 7, host + 40 * MIB, n, bm.BmCopyType.G2G) == 0
        assert np.array_equal(hview[40 * MIB:40 * MIB + n], payload)
        assert pool.copy_data(host + 40 * MIB, dev + 64 * MIB + 3, n, bm.BmCopyType.G2G) == 0
        got = np.empty(n, dtype=np.uint8)
        assert lib.mfrt_memcpy(np_ptr(got), dev + 64 * MIB + 3, n) == 0
        assert np.array_equal(got, payload)
        # L2GH / GH2L do not override a side: a local address is unclassifiable -> invalid param
        assert pool.copy_data(local_dev.ptr, host, n, bm.BmCopyType.L2GH) == native.SM_INVALID_PARAM
        assert pool.copy_data(host, local_dev.ptr, n, bm.BmCopyType.GH2L) == native.SM_INVALID_PARAM
    finally:
        local_dev.free()
        pinned.free()


def test_pageable_batches_go_through_staging(pool, lib, oracle):
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    count = 40
    rng = np.random.default_rng(5)
    lens = rng.integers(1, 2 * MIB, count)
    lens[3] = 40 * MIB  # larger than the staging area: cut into rounds
    total = int(lens.sum())
    payload = _rand(oracle, total, 0xD3)
    offs = np.concatenate([[0], np.cumsum(lens)[:-1]])
    assert total + count * 64 <= POOL
    dst = dev + offs + np.arange(count) * 64 + 1
    assert pool.copy_data_batch((np_ptr(payload) + offs).tolist(), dst.tolist(), lens.tolist(), count,
                                bm.BmCopyType.H2G) == 0, native.last_error()
    landed = np.empty(total + count * 64 + 1, dtype=np.uint8)     # what is in the pool now, read by plain hipMemcpy
    assert lib.mfrt_memcpy(np_ptr(landed), dev, len(landed)) == 0
    for i in range(count):
        at = int(offs[i]) + i * 64 + 1
        assert np.array_equal(landed[at:at + int(lens[i])], payload[int(offs[i]):int(offs[i]) + int(lens[i])]), i
    back = np.zeros(total, dtype=np.uint8)
    assert pool.copy_data_batch(dst.tolist(), (np_ptr(back) + offs).tolist(), lens.tolist(), count,
                                bm.BmCopyType.G2H) == 0
    assert np.array_equal(back, payload)


def test_pageable_copy_that_wraps_the_ring_of_small_slots(pool, lib, oracle):
    """48 MiB is below the size that switches to large staging slots and above what the ring of
    small ones holds, so slots are reused in both directions."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    n = 48 * MIB + 5
    payload = _rand(oracle, n, 0xD4)
    assert pool.copy_data(np_ptr(payload), dev + 3, n, bm.BmCopyType.H2G) == 0, native.last_error()
    back = np.zeros(n, dtype=np.uint8)
    assert pool.copy_data(dev + 3, np_ptr(back), n, bm.BmCopyType.G2H) == 0
    assert np.array_equal(back, payload)


def test_reference_example_pattern_round_trip(pool, lib, oracle):
    """The check the reference's own example performs (example/bm/BmCpp/main.cpp:142-197 of the
    reference): fill with the LCG pattern, copy host -> pool -> host, compare word by word."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    n = 8 * MIB
    for rank in (0, 1, 5):
        src = np.zeros(n, dtype=np.uint8)
        oracle.orc_lcg_fill(np_ptr(src), rank, n)
        assert pool.copy_data(np_ptr(src), dev, n, bm.BmCopyType.H2G) == 0
        out = np.zeros(n, dtype=np.uint8)
        assert pool.copy_data(dev, np_ptr(out), n, bm.BmCopyType.G2H) == 0
        assert oracle.orc_lcg_mismatch(np_ptr(src), np_ptr(out), n) == 0


def test_async_copy_completes_on_wait(pool, lib, oracle):
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    n = 32 * MIB
    block = _rand(oracle, n, 0xD4)
    assert lib.mfrt_memcpy(dev, np_ptr(block), n) == 0
    for i in range(3):  # three queued copies chained through the pool, then one wait
        assert pool.copy_data(dev + i * n, dev + (i + 1) * n, n, bm.BmCopyType.G2G, native.ASYNC_COPY_FLAG) == 0
    assert pool.wait() == 0
    got = np.empty(n, dtype=np.uint8)
    assert lib.mfrt_memcpy(np_ptr(got), dev + 3 * n, n) == 0
    assert np.array_equal(got, block)


@pytest.mark.parametrize("side_streams", [0, 2, 6])
def test_unordered_batches_and_the_ordered_copy_behind_them(pool, lib, oracle, side_streams):
    """MF_COPY_UNORDERED_FLAG: batches the caller declares independent are launched without a barrier on the
    thread's stream, or (mf_xcopy_unordered_streams) handed in turn to submit threads of the library's.
    Sixty such batches of up to 100 ragged pieces, all with destinations of their own, then ONE ordinary
    asynchronous copy that reads what they wrote: it has to wait for all of them.  Compared with the
    oracle applied in order; repeated so that an ordering slip has many chances to show.  The last round
    ends in smem_bm_wait alone, which has to cover the submit threads' streams as well."""
    assert lib.mf_xcopy_unordered_streams(side_streams) == 0
    try:
        _unordered_then_ordered(pool, lib, oracle)
    finally:
        assert lib.mf_xcopy_unordered_streams(0) == 0
    assert lib.mf_xcopy_unordered_streams(9) == native.BM_INVALID_PARAM


def _unordered_then_ordered(pool, lib, oracle):
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    half = 40 * MIB
    init = _rand(oracle, half, 0xD8)
    g2g = bm.BmCopyType.G2G
    flags = native.ASYNC_COPY_FLAG | native.MF_COPY_UNORDERED_FLAG
    rng = np.random.default_rng(12)
    got = np.empty(half, dtype=np.uint8)
    for rep in range(4):
        assert lib.mfrt_memcpy(dev, np_ptr(init), half) == 0
        assert lib.mfrt_memset(dev + half, 0x11 + rep, 2 * half) == 0
        expect = np.full(half, 0x11 + rep, dtype=np.uint8)
        cursor = 0
        for b in range(60):
            count = int(rng.integers(1, 101))
            lens = rng.integers(0, 20000, count)
            src = rng.integers(0, half - 20000, count)
            dst = cursor + np.cumsum(lens + 13) - lens - 13          # disjoint destinations, 13 bytes apart, any alignment
            cursor = int(dst[-1] + lens[-1] + 13)
            assert cursor < half
            assert pool.copy_data_batch((dev + src).tolist(), (dev + half + dst).tolist(), lens.tolist(), count, g2g, flags) == 0, \
                native.last_error()
            gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
        # ordinary (ordered) copy of everything the unordered batches wrote
        assert pool.copy_data(dev + half, dev + 2 * half, half, g2g, native.ASYNC_COPY_FLAG) == 0, native.last_error()
        assert pool.wait() == 0
        assert lib.mfrt_memcpy(np_ptr(got), dev + 2 * half, half) == 0
        assert np.array_equal(got, expect), rep
    # unordered batches and nothing but the wait behind them
    assert lib.mfrt_memset(dev + half, 0x77, half) == 0
    expect = np.full(half, 0x77, dtype=np.uint8)
    cursor = 0
    for b in range(40):
        count = int(rng.integers(1, 101))
        lens = rng.integers(0, 20000, count)
        src = rng.integers(0, half - 20000, count)
        dst = cursor + np.cumsum(lens + 13) - lens - 13
        cursor = int(dst[-1] + lens[-1] + 13)
        assert pool.copy_data_batch((dev + src).tolist(), (dev + half + dst).tolist(), lens.tolist(), count, g2g, flags) == 0, \
            native.last_error()
        gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
    assert pool.wait() == 0
    assert lib.mfrt_memcpy(np_ptr(got), dev + half, half) == 0
    assert np.array_equal(got, expect)


def test_held_stores_copy_the_same_bytes(pool, lib, oracle):
    """Batches of 1000 to 5600 chunks wait with their stores (mf_xcopy_hold_stores).  Three ragged batches
    of that size, each reading what the one before wrote, cycled on one stream, with the library's rule,
    with no wait and with a wait far longer than any load takes: the same bytes as the oracle applied in
    order every time (pieces start and end at any byte, so waves with partial chunks wait too)."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    region = 12 * MIB
    n = 3 * region
    init = _rand(oracle, n, 0xD9)
    rng = np.random.default_rng(13)
    tables = []
    for b in range(3):   # batch b moves 48 ragged pieces (about 7 MB, 1800 chunks) from region b to region (b + 1) % 3
        lens = rng.integers(100000, 200000, 48)
        src = b * region + np.cumsum(lens) - lens + rng.integers(0, 7)
        dst = ((b + 1) % 3) * region + np.cumsum(lens) - lens + rng.integers(0, 7)
        assert int(lens.sum()) + 7 < region
        tables.append((src, dst, lens))
    g2g = bm.BmCopyType.G2G
    got = np.empty(n, dtype=np.uint8)
    try:
        for nanos in (-1, 0, 9000):
            assert lib.mf_xcopy_hold_stores(nanos) == 0
            assert lib.mfrt_memcpy(dev, np_ptr(init), n) == 0
            expect = init.copy()
            for step in range(7):
                src, dst, lens = tables[step % 3]
                assert pool.copy_data_batch((dev + src).tolist(), (dev + dst).tolist(), lens.tolist(), len(lens), g2g,
                                            native.ASYNC_COPY_FLAG) == 0, native.last_error()
                before = expect.copy()
                gpu_util.oracle_batch(oracle, before, expect, src, dst, lens)
            assert pool.wait() == 0
            assert lib.mfrt_memcpy(np_ptr(got), dev, n) == 0
            assert np.array_equal(got, expect), nanos
    finally:
        assert lib.mf_xcopy_hold_stores(-1) == 0
    assert lib.mf_xcopy_hold_stores(-2) != 0


def test_replayed_batches_keep_stream_order(pool, lib, oracle):
    """mf_bm_copy_batch_replay issues the same calls a loop would: three batches, each reading what
    the one before wrote, cycled for seven steps on one stream, against the oracle applied in order."""
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    n = 24 * MIB
    init = _rand(oracle, n, 0xD6)
    assert lib.mfrt_memcpy(dev, np_ptr(init), n) == 0
    region = 8 * MIB
    rng = np.random.default_rng(11)
    tables = []
    for b in range(3):   # batch b moves 40 ragged pieces from region b to region (b + 1) % 3
        lens = rng.integers(1, 150000, 40)
        src = b * region + np.cumsum(lens) - lens + rng.integers(0, 7)
        dst = ((b + 1) % 3) * region + np.cumsum(lens) - lens + rng.integers(0, 7)
        tables.append((src, dst, lens))
    keep = []
    blocks = []
    for src, dst, lens in tables:
        srcs = native.ptr_array((dev + src).tolist())
        dsts = native.ptr_array((dev + dst).tolist())
        sizes = native.u64_array(lens.tolist())
        params = native.BatchCopyParams(srcs, dsts, sizes, len(lens))
        keep.append((srcs, dsts, sizes))
        blocks.append(params)
    table = (ctypes.POINTER(native.BatchCopyParams) * 3)(*[ctypes.pointer(p) for p in blocks])
    steps = 7
    assert lib.mf_bm_copy_batch_replay(pool.handle, table, 3, steps, int(bm.BmCopyType.G2G),
                                       native.ASYNC_COPY_FLAG) == 0, native.last_error()
    assert pool.wait() == 0
    expect = init.copy()
    for i in range(steps):
        src, dst, lens = tables[i % 3]
        before = expect.copy()
        gpu_util.oracle_batch(oracle, before, expect, src, dst, lens)
    got = np.empty(n, dtype=np.uint8)
    assert lib.mfrt_memcpy(np_ptr(got), dev, n) == 0
    assert np.array_equal(got, expect)
    assert lib.mf_bm_copy_batch_replay(pool.handle, None, 3, 1, int(bm.BmCopyType.G2G), 0) == native.SM_INVALID_PARAM
    assert lib.mf_bm_copy_batch_replay(pool.handle, table, 3, 0, int(bm.BmCopyType.G2G), 0) == 0


def test_range_and_argument_errors(pool, lib):
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    host = pool.peer_rank_ptr(0, bm.BmMemType.HOST)
    G2G = bm.BmCopyType.G2G
    assert pool.copy_data(dev, dev + POOL - 8, 16, G2G) == native.SM_INVALID_PARAM      # leaves the window
    assert pool.copy_data(0, dev, 16, G2G) == native.SM_INVALID_PARAM
    assert pool.copy_data(dev, 0, 16, G2G) == native.SM_INVALID_PARAM
    assert pool.copy_data(dev, host, 0, G2G) == native.SM_INVALID_PARAM
    assert pool.copy_data(dev, host, 16, 10) == native.SM_INVALID_PARAM                  # BUTT
    assert pool.copy_data_batch([dev, 0], [host, host + 64], [16, 16], 2, G2G) == native.BM_INVALID_PARAM
    assert pool.copy_data_batch([dev, dev], [host, host + POOL], [16, 16], 2, G2G) == native.BM_INVALID_PARAM
    assert pool.copy_data_batch([dev], [host], [0], 1, G2G) == 0                         # zero length is a no-op
    assert lib.smem_bm_create(3, 1, 1, 2 * MIB, 2 * MIB, 0) is None                      # duplicate id
    assert lib.smem_bm_create(4, 1, 1, 2 * MIB + 5, 0, 0) is None                        # not 2 MiB granular
    assert lib.smem_bm_create(5, 1, 0, 2 * MIB, 2 * MIB, 0) is None                      # no data op type


def test_plugin_abi(pool, lib, oracle):
    """hybm_copy_extend / hybm_batch_copy_extend as the reference calls them
    (hybm_data_op_sdma.cpp:419-425,504-543 of the reference): pinned parameter table, completion word."""
    plug = native.plugin()
    dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
    n = 16 * MIB
    init = _rand(oracle, n, 0xD5)
    assert lib.mfrt_memcpy(dev, np_ptr(init), n) == 0
    stream = lib.mfrt_stream_create()
    params = gpu_util.PinnedBuffer(lib, 16384 * 24 + 64)
    table_dev = gpu_util.DeviceBuffer(lib, 16384 * 24)
    try:
        plug.hybm_copy_extend(dev + 3, dev + 64 * MIB + 1, n - 3, 32, stream)
        assert lib.mfrt_stream_sync(stream) == 0
        got = np.empty(n - 3, dtype=np.uint8)
        assert lib.mfrt_memcpy(np_ptr(got), dev + 64 * MIB + 1, n - 3) == 0
        assert np.array_equal(got, init[3:])

        for count in (122, 3000):
            src, dst, lens = workloads.ragged_batch(count, n, count, max_len=4000 if count > 200 else 60000)
            triples = np.empty((count, 3), dtype=np.uint64)
            triples[:, 0] = dev + src
            triples[:, 1] = dev + 96 * MIB + dst
            triples[:, 2] = lens
            raw = triples.view(np.uint8).reshape(-1)
            params.array[:len(raw)] = raw
            mask = params.array[16384 * 24:16384 * 24 + 8].view(np.uint64)
            mask[0] = 0
            assert lib.mfrt_memset(dev + 96 * MIB, 0x44, n) == 0
            plug.hybm_batch_copy_extend(params.ptr, count, params.ptr + 16384 * 24, 32, stream)
            assert lib.mfrt_stream_sync(stream) == 0
            assert mask[0] == 32
            got = np.empty(n, dtype=np.uint8)
            assert lib.mfrt_memcpy(np_ptr(got), dev + 96 * MIB, n) == 0
            expect = np.full(n, 0x44, dtype=np.uint8)
            gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
            assert np.array_equal(got, expect)

            # the same table resident in device memory, completion word in pinned memory
            table_dev.upload(raw)
            mask[0] = 0
            assert lib.mfrt_memset(dev + 96 * MIB, 0x45, n) == 0
            plug.hybm_batch_copy_extend(table_dev.ptr, count, params.ptr + 16384 * 24, 32, stream)
            assert lib.mfrt_stream_sync(stream) == 0
            assert mask[0] == 32
            assert lib.mfrt_memcpy(np_ptr(got), dev + 96 * MIB, n) == 0
            expect = np.full(n, 0x45, dtype=np.uint8)
            gpu_util.oracle_batch(oracle, init, expect, src, dst, lens)
            assert np.array_equal(got, expect)
    finally:
        params.free()
        table_dev.free()
        lib.mfrt_stream_destroy(stream)


def test_launch_cost_per_cpu_and_pinning_near_the_gpu(lib, pool):
    """Every CPU of the thread's set is measured and the set is put back; the pinned set is a part of it and copies
    still work from there."""
    import os
    before = os.sched_getaffinity(0)
    cpus, micros = (ctypes.c_uint32 * 1024)(), (ctypes.c_float * 1024)()
    n = lib.mf_host_launch_costs(cpus, micros, 1024)
    assert n == len(before), native.last_error()
    assert os.sched_getaffinity(0) == before
    assert {int(cpus[i]) for i in range(n)} == set(before)
    assert all(0.5 < float(micros[i]) < 100.0 for i in range(n)), [float(micros[i]) for i in range(n)]
    try:
        kept = lib.mf_pin_thread_near_gpu()
        assert 1 <= kept <= n
        near = os.sched_getaffinity(0)
        assert len(near) == kept and near <= before
        src = gpu_util.DeviceBuffer(lib, 1 << 20)
        dst = gpu_util.DeviceBuffer(lib, 1 << 20)
        data = np.random.default_rng(5).integers(0, 256, 1 << 20, dtype=np.uint8)
        src.upload(data)
        s, d, l = native.u64_array([src.ptr]), native.u64_array([dst.ptr]), native.u64_array([1 << 20])
        assert lib.mf_xcopy_batch(s, d, l, 1, native.ROUTE_HBM, None) == 0
        assert lib.mfrt_device_sync() == 0
        assert np.array_equal(dst.download(0, 1 << 20), data)
        src.free()
        dst.free()
    finally:
        os.sched_setaffinity(0, before)


def test_start_up_check_of_the_timing_rules(lib, pool):
    """hybm_init has timed the held stores and the read and write windows on this GPU: the seven times are there and
    plausible for an MI355X, and what it chose is one of the settings it tried."""
    enabled, delta, rate, aligned_rate = ctypes.c_int32(-7), ctypes.c_int32(-7), ctypes.c_uint32(7), ctypes.c_uint32(7)
    long_rate = ctypes.c_uint32(7)
    micros = (ctypes.c_float * 8)()
    ran = lib.mf_xcopy_calibration(ctypes.byref(enabled), ctypes.byref(delta), ctypes.byref(rate), ctypes.byref(aligned_rate), ctypes.byref(long_rate), micros)
    if ran == 0:
        pytest.skip("MF_HIP_CALIBRATE=0 in this environment")
    times = [float(t) for t in micros]
    assert all(1.0 < t < 60.0 for t in times[:4]), times          # a 9 MB batch
    assert all(100.0 < t < 2000.0 for t in times[4:]), times      # a 512 MiB copy
    assert enabled.value in (0, 1) and delta.value in (-200, 0, 200)
    assert rate.value in (0, 6800000, 6800000 * 94 // 100)
    assert (aligned_rate.value, long_rate.value) in ((rate.value, rate.value), (7100000, 7400000))
    assert rate.value != 0 or aligned_rate.value == 0
    if enabled.value == 1:
        chosen = {0: times[1], -200: times[2], 200: times[3]}[delta.value]
        assert chosen <= times[0] * 0.97 + 1e-3, times             # holding gained its 3 %
