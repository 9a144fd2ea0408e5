"""GPU tests of the transfer front-end (smem_trans_* and its TransferEngine mirror): a "Prefill"
object writes KV-shaped batches into memory a "Decode" object registered, both in this process on
the one GPU, and the bytes are compared with the oracle's memcpy loop.  The flow is the one of
the reference's two-process tests (test/ut/testcase/smem/smem_trans_test.cpp:272-373,655-779) and
of its demo (example/trans/demo/test_transfer_engine.py)."""

import ctypes

import numpy as np
import pytest

from memfabric_hybrid_amd import native, workloads
from memfabric_hybrid_amd.transfer import TransferEngine
from tests import gpu_util
from tests.oracle_lib import np_ptr

pytestmark = pytest.mark.gpu

MIB = 1 << 20
POOL = 96 * MIB
PREFILL = "127.0.0.1:15321"
DECODE = "127.0.0.1:15322"
STORE = "tcp://127.0.0.1:15432"


@pytest.fixture(scope="module")
def engines(lib):
    prefill, decode = TransferEngine(), TransferEngine()
    assert prefill.initialize(STORE, PREFILL, "Prefill", 0) == 0, native.last_error()
    assert decode.initialize(STORE, DECODE, "Decode", 0) == 0, native.last_error()
    assert TransferEngine().initialize(STORE, "127.0.0.1:15399", "Other", 0) == -1
    yield prefill, decode
    prefill.destroy()
    decode.destroy()
    prefill.unInitialize()


def _random(oracle, nbytes, seed):
    a = np.empty(nbytes, dtype=np.uint8)
    oracle.orc_fill_random(np_ptr(a), nbytes, seed)
    return a


def test_kv_batch_write_then_read(lib, oracle, engines):
    prefill, decode = engines
    local = gpu_util.DeviceBuffer(lib, POOL)
    remote = gpu_util.DeviceBuffer(lib, POOL)
    back = gpu_util.DeviceBuffer(lib, POOL)
    try:
        data = _random(oracle, POOL, 0x7101)
        local.upload(data)
        remote.fill(0)
        back.fill(0)
        assert decode.register_memory(remote.ptr, POOL) == 0, native.last_error()
        src, dst, lens = workloads.kv_batch(0x7102, POOL, POOL, same_pool=False)
        launches = lib.mf_xcopy_launch_count()
        ret = prefill.batch_transfer_sync_write(DECODE, [local.ptr + int(s) for s in src],
                                                [remote.ptr + int(d) for d in dst], [int(n) for n in lens])
        assert ret == 0, native.last_error()
        assert lib.mf_xcopy_launch_count() == launches + 1        # the whole batch is one launch
        want = np.zeros(POOL, dtype=np.uint8)
        gpu_util.oracle_batch(oracle, data, want, src, dst, lens)
        assert np.array_equal(remote.download(), want)
        # read the same segments back to where they came from, in a fresh buffer
        ret = prefill.batch_transfer_sync_read(DECODE, [back.ptr + int(s) for s in src],
                                               [remote.ptr + int(d) for d in dst], [int(n) for n in lens])
        assert ret == 0, native.last_error()
        want_back = np.zeros(POOL, dtype=np.uint8)
        gpu_util.oracle_batch(oracle, data, want_back, src, src, lens)
        assert np.array_equal(back.download(), want_back)
        # a range that leaves the registered memory is refused before anything is launched
        launches = lib.mf_xcopy_launch_count()
        assert prefill.transfer_sync_write(DECODE, local.ptr, remote.ptr + POOL - 8, 16) == native.SM_INVALID_PARAM
        assert prefill.transfer_sync_write(PREFILL, local.ptr, remote.ptr, 16) == native.SM_INVALID_PARAM
        assert lib.mf_xcopy_launch_count() == launches
        assert decode.unregister_memory(remote.ptr) == 0
        assert prefill.transfer_sync_write(DECODE, local.ptr, remote.ptr, 16) == native.SM_INVALID_PARAM
    finally:
        local.free()
        remote.free()
        back.free()


def test_ragged_batches_all_memory_kinds(lib, oracle, engines):
    """Unaligned lengths and offsets; the peer's memory is HBM or pinned host memory the object
    allocated itself; the local side is HBM, pinned or ordinary pageable memory."""
    prefill, decode = engines
    nbytes = 8 * MIB
    handle = decode._handle
    peer_host = lib.smem_trans_malloc(handle, nbytes - 5)           # rounded up to 2 MiB pages
    assert peer_host, native.last_error()
    peer_dev = gpu_util.DeviceBuffer(lib, nbytes)
    local_dev = gpu_util.DeviceBuffer(lib, nbytes)
    local_pin = gpu_util.PinnedBuffer(lib, nbytes)
    local_page = np.zeros(nbytes, dtype=np.uint8)
    try:
        assert decode.register_memory(peer_dev.ptr, nbytes) == 0
        data = _random(oracle, nbytes, 0x7201)
        local_dev.upload(data)
        local_pin.array[:] = data
        local_page[:] = data
        src, dst, lens = workloads.ragged_batch(0x7202, nbytes, 300, max_len=20000)
        want = np.zeros(nbytes, dtype=np.uint8)
        keep = lens > 0                                             # the front-end refuses empty elements
        src, dst, lens = src[keep], dst[keep], lens[keep]
        gpu_util.oracle_batch(oracle, data, want, src, dst, lens)
        locals_ = {"hbm": local_dev.ptr, "pinned": local_pin.ptr, "pageable": np_ptr(local_page)}
        for peer_name, peer in (("hbm", peer_dev.ptr), ("host", peer_host)):
            for local_name, base in locals_.items():
                if peer_name == "hbm":
                    peer_dev.fill(0)
                else:
                    ctypes.memset(peer_host, 0, nbytes)
                ret = prefill.batch_transfer_sync_write(DECODE, [base + int(s) for s in src],
                                                        [peer + int(d) for d in dst], [int(n) for n in lens])
                assert ret == 0, (peer_name, local_name, native.last_error())
                got = peer_dev.download() if peer_name == "hbm" else gpu_util.host_view(peer_host, nbytes).copy()
                assert np.array_equal(got, want), (peer_name, local_name)
        with_zero = [int(n) for n in lens]
        with_zero[3] = 0
        assert prefill.batch_transfer_sync_write(DECODE, [local_dev.ptr + int(s) for s in src],
                                                 [peer_dev.ptr + int(d) for d in dst], with_zero) == native.SM_INVALID_PARAM
        assert lib.smem_trans_free(handle, peer_host) == 0
        assert prefill.transfer_sync_write(DECODE, local_dev.ptr, peer_host, 16) == native.SM_INVALID_PARAM
        assert decode.unregister_memory(peer_dev.ptr) == 0
    finally:
        peer_dev.free()
        local_dev.free()
        local_pin.free()


def test_submit_on_a_torch_stream_is_ordered_after_the_producer(lib, engines):
    """The hazard the reference documents in test/python/tensor/copy_consistency_test.py: a tensor
    produced on one stream and copied on another may be copied before it exists.  Submitting on
    the producer's stream orders the copy after it; sums of source and copy must agree."""
    torch = pytest.importorskip("torch")
    prefill, decode = engines
    n = 32 * MIB
    stream = torch.cuda.Stream(device=0)
    landing = torch.zeros(n // 2, dtype=torch.float16, device="cuda:0")
    returned = torch.zeros(n // 2, dtype=torch.float16, device="cuda:0")
    torch.cuda.synchronize()
    assert decode.register_memory(landing.data_ptr(), n) == 0, native.last_error()
    try:
        for _ in range(5):
            with torch.cuda.stream(stream):
                produced = torch.rand(n // 2, dtype=torch.float32, device="cuda:0").to(torch.float16)
                assert prefill.transfer_async_write_submit(DECODE, produced.data_ptr(), landing.data_ptr(), n,
                                                           stream.cuda_stream) == 0, native.last_error()
                assert prefill.transfer_async_read_submit(DECODE, returned.data_ptr(), landing.data_ptr(), n,
                                                          stream.cuda_stream) == 0, native.last_error()
                total_src = produced.sum(dtype=torch.float32)
                total_dst = returned.sum(dtype=torch.float32)
            stream.synchronize()
            assert total_src.item() == total_dst.item() and total_src.item() > 0
            assert torch.equal(produced, returned)
    finally:
        assert decode.unregister_memory(landing.data_ptr()) == 0
