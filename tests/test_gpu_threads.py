"""Concurrent callers on the GPU: eight host threads, each on its own stream and its own slice of
one pool, mix small batches (descriptors in the kernel arguments), large batches (descriptor table
staged through the thread's slot ring), pageable host memory (staging ring) and transfer-object
writes, every result compared with the oracle.  A second generation of threads then reuses the
streams and staging memory the first one handed back.  The reference serves concurrent callers the
same way, one stream per calling thread (src/hybm/csrc/ts_engine/hybm_stream_manager.cpp:73-90)."""

import threading

import numpy as np
import pytest

from memfabric_hybrid_amd import bm, native, workloads
from memfabric_hybrid_amd.transfer import TransferEngine
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

MIB = 1 << 20
THREADS = 8
SLICE = 32 * MIB                 # per thread: lower half sources, upper half destinations
POOL = THREADS * SLICE
DECODE = "127.0.0.1:16322"


def _worker(tid, generation, lib, oracle, pool, prefill, data, errors):
    try:
        assert lib.mfrt_bind_thread() == 0
        dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE) + tid * SLICE
        mine = data[tid * SLICE:(tid + 1) * SLICE]
        half = SLICE // 2
        scratch = np.zeros(half, dtype=np.uint8)          # ordinary pageable memory of this thread
        for step in range(6):
            seed = 0x7000 + generation * 1000 + tid * 10 + step
            count = (100, 700, 60, 122, 3000, 40)[step]
            src, dst, lens = workloads.ragged_batch(seed, SLICE, count, max_len=(SLICE // 4) // count)
            want = np.zeros(half, dtype=np.uint8)
            assert lib.mfrt_memset(dev + half, 0, half) == 0
            kind = step % 3
            if kind == 0:      # pool to pool, asynchronous, then wait
                gpu_util.oracle_batch(oracle, mine, want, src, dst - half, lens)
                ret = pool.copy_data_batch((dev + src).tolist(), (dev + dst).tolist(), lens.tolist(), count,
                                           bm.BmCopyType.G2G, native.ASYNC_COPY_FLAG)
                assert ret == 0, native.last_error()
                assert pool.wait() == 0
            elif kind == 1:    # pageable host memory into the pool and out again
                scratch[:] = mine[:half]
                gpu_util.oracle_batch(oracle, scratch, want, src, dst - half, lens)
                ret = pool.copy_data_batch((np_ptr(scratch) + src).tolist(), (dev + dst).tolist(), lens.tolist(), count,
                                           bm.BmCopyType.H2G)
                assert ret == 0, native.last_error()
                back = np.zeros(half, dtype=np.uint8)
                ret = pool.copy_data_batch((dev + dst).tolist(), (np_ptr(back) + (dst - half)).tolist(), lens.tolist(),
                                           count, bm.BmCopyType.G2H)
                assert ret == 0, native.last_error()
                assert np.array_equal(back, want), f"thread {tid} step {step}: read back through staging differs"
            else:              # transfer-object write into the registered pool
                keep = lens > 0
                gpu_util.oracle_batch(oracle, mine, want, src[keep], dst[keep] - half, lens[keep])
                ret = prefill.batch_transfer_sync_write(DECODE, (dev + src[keep]).tolist(), (dev + dst[keep]).tolist(),
                                                        lens[keep].tolist())
                assert ret == 0, native.last_error()
            got = np.empty(half, dtype=np.uint8)
            assert lib.mfrt_memcpy(np_ptr(got), dev + half, half) == 0
            assert np.array_equal(got, want), f"thread {tid} generation {generation} step {step} kind {kind}"
    except BaseException as exc:  # noqa: BLE001
        errors.append((tid, generation, repr(exc)))


def test_eight_threads_two_generations(lib, oracle):
    assert bm.initialize("tcp://127.0.0.1:5432", 1, 0) == 0, native.last_error()
    pool = bm.create(9, 0, POOL, bm.BmDataOpType.SDMA)
    prefill, decode = TransferEngine(), TransferEngine()
    try:
        assert pool.join() == 0
        dev = pool.peer_rank_ptr(0, bm.BmMemType.DEVICE)
        data = np.empty(POOL, dtype=np.uint8)
        oracle.orc_fill_random(np_ptr(data), POOL, 0x7EAD)
        assert lib.mfrt_memcpy(dev, np_ptr(data), POOL) == 0
        assert prefill.initialize("tcp://127.0.0.1:16432", "127.0.0.1:16321", "Prefill", 0) == 0
        assert decode.initialize("tcp://127.0.0.1:16432", DECODE, "Decode", 0) == 0
        assert decode.register_memory(dev, POOL) == 0, native.last_error()
        launches = lib.mf_xcopy_launch_count()
        for generation in range(2):
            errors = []
            threads = [threading.Thread(target=_worker, args=(t, generation, lib, oracle, pool, prefill, data, errors))
                       for t in range(THREADS)]
            for t in threads:
                t.start()
            for t in threads:
                t.join(timeout=100)
            assert not any(t.is_alive() for t in threads), "a worker is stuck"
            assert not errors, errors
            # sources were never written: the lower halves still hold the original bytes
            check = np.empty(SLICE // 2, dtype=np.uint8)
            for t in range(THREADS):
                assert lib.mfrt_memcpy(np_ptr(check), dev + t * SLICE, SLICE // 2) == 0
                assert np.array_equal(check, data[t * SLICE:t * SLICE + SLICE // 2]), t
        assert lib.mf_xcopy_launch_count() > launches
        assert decode.unregister_memory(dev) == 0
    finally:
        prefill.destroy()
        decode.destroy()
        prefill.unInitialize()
        pool.destroy()
        bm.uninitialize()


def _chain_worker(tid, lib, dev, data, errors):
    """24 asynchronous table batches in a row, each reading what the one before wrote: page
    permutations (descriptors read from the staging slot while the kernel runs) take turns with ragged
    batches (table uploaded first).  The host runs ahead of the GPU, so the staging ring wraps while
    kernels still read it; a slot rewritten too early would scramble a later batch."""
    try:
        assert lib.mfrt_bind_thread() == 0
        region = 32 * MIB
        base = dev + tid * 3 * region
        model = [data[(tid * 3 + r) * region:(tid * 3 + r + 1) * region].copy() for r in range(3)]
        rng = np.random.default_rng(0x600 + tid)
        keep = []
        for step in range(24):
            s_reg, d_reg = step % 3, (step + 1) % 3
            if step % 2 == 0:
                page = 16384
                pages = region // page
                order = rng.permutation(pages)
                src = order.astype(np.uint64) * page
                dst = np.arange(pages, dtype=np.uint64) * page
                lens = np.full(pages, page, dtype=np.uint64)
                model[d_reg] = model[s_reg].reshape(pages, page)[order].reshape(-1).copy()
            else:
                count = 1500
                slot = region // count
                lens = rng.integers(1, slot, count).astype(np.uint64)
                src = rng.permutation(count).astype(np.uint64) * slot
                dst = np.arange(count, dtype=np.uint64) * slot
                out = model[d_reg].copy()
                for i in range(count):
                    out[int(dst[i]):int(dst[i]) + int(lens[i])] = model[s_reg][int(src[i]):int(src[i]) + int(lens[i])]
                model[d_reg] = out
            arrays = (native.u64_array((base + s_reg * region + src).tolist()),
                      native.u64_array((base + d_reg * region + dst).tolist()), native.u64_array(lens.tolist()))
            keep.append((arrays, len(lens)))
        for arrays, count in keep:   # all at once: the host finishes queueing long before the GPU is through
            assert lib.mf_xcopy_batch(arrays[0], arrays[1], arrays[2], count, native.ROUTE_HBM, None) == 0, native.last_error()
        assert lib.mfrt_stream_sync(lib.mf_xcopy_thread_stream()) == 0
        got = np.empty(region, dtype=np.uint8)
        for r in range(3):
            assert lib.mfrt_memcpy(np_ptr(got), base + r * region, region) == 0
            assert np.array_equal(got, model[r]), f"thread {tid} region {r}"
    except BaseException as exc:  # noqa: BLE001
        errors.append((tid, repr(exc)))


def test_table_batches_in_a_row_keep_their_descriptors(lib, oracle):
    threads_n = 3
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    total = threads_n * 3 * 32 * MIB
    buf = gpu_util.DeviceBuffer(lib, total)
    try:
        data = np.empty(total, dtype=np.uint8)
        oracle.orc_fill_random(np_ptr(data), total, 0x7EAE)
        buf.upload(data)
        errors = []
        threads = [threading.Thread(target=_chain_worker, args=(t, lib, buf.ptr, data, errors)) for t in range(threads_n)]
        for t in threads:
            t.start()
        for t in threads:
            t.join(timeout=100)
        assert not any(t.is_alive() for t in threads), "a worker is stuck"
        assert not errors, errors
    finally:
        buf.free()
        lib.hybm_uninit()


def test_streams_are_dealt_one_per_hardware_queue(lib):
    """hybm_init classifies the streams it makes by hardware queue and hands out one of every queue before the second of
    any.  Checked against a measurement of its own through the public calls: a long copy on one stream, a short one on
    another, and whether the short one ends first."""
    import ctypes
    assert lib.hybm_init(0, 0) == 0, native.last_error()
    try:
        queues = (ctypes.c_uint32 * 16)()
        count = lib.mf_xcopy_stream_queues(queues, 16)
        assert count == 8
        dealt = list(queues[:count])
        kinds = len(set(dealt))
        assert kinds >= 2, "the runtime of an MI355X spreads its streams over several hardware queues"
        assert sorted(dealt[:kinds]) == list(range(kinds)), dealt      # the first round: one stream of every queue
        # the calling thread holds the deck's first stream; a second thread gets the second, which must overlap with it
        mine = lib.mf_xcopy_thread_stream()
        other = []

        def grab():
            assert lib.mfrt_bind_thread() == 0
            other.append(lib.mf_xcopy_thread_stream())

        t = threading.Thread(target=grab)
        t.start()
        t.join()
        assert other and other[0] and other[0] != mine
        big = 256 * MIB
        buf = gpu_util.DeviceBuffer(lib, 2 * big + 8192)
        ea, eb = lib.mfrt_event_create(), lib.mfrt_event_create()
        u64 = ctypes.c_uint64
        try:
            def copy(stream, src, dst, n):
                assert lib.mf_xcopy_batch((u64 * 1)(src), (u64 * 1)(dst), (u64 * 1)(n), 1, native.ROUTE_HBM, stream) == 0
            for s in (mine, other[0]):
                copy(s, buf.ptr, buf.ptr + big, 4096)
            assert lib.mfrt_device_sync() == 0
            overlapped = 0
            for _ in range(5):
                copy(mine, buf.ptr, buf.ptr + big, big)                       # some 90 us
                lib.mfrt_event_record(ea, mine)
                copy(other[0], buf.ptr + 2 * big, buf.ptr + 2 * big + 4096, 4096)
                lib.mfrt_event_record(eb, other[0])
                assert lib.mfrt_event_sync(eb) == 0
                overlapped += 0 if lib.mfrt_event_done(ea) else 1
                assert lib.mfrt_event_sync(ea) == 0
            assert overlapped >= 4, "the second thread's stream waits for the first thread's copies"
            # the library's own probe says the same, and knows a stream shares a queue with itself
            assert lib.mfrt_device_sync() == 0
            assert lib.mfrt_streams_share_queue(mine, other[0]) == 0
            assert lib.mfrt_streams_share_queue(mine, mine) == 1
        finally:
            lib.mfrt_event_destroy(ea)
            lib.mfrt_event_destroy(eb)
            buf.free()
    finally:
        lib.hybm_uninit()
